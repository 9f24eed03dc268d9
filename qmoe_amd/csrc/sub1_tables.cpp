// Host-side builder of the fixed QMoE dictionary (decode table + encode trie).
//
// Reference: sub1.py:29-102 builds the same two arrays in Python with a heap.
// Here the dictionary is produced from its closed form instead: the heap there
// pops strings of pair symbols in increasing order of
//   (negated probability as an IEEE double product taken left to right,
//    then the string itself, lexicographically, a proper prefix first),
// because every extension of a string has a strictly larger key than the
// string.  So the dictionary is the first 65536 strings of 1..14 pairs under
// that order.  We enumerate every string whose key lies below a cut, sort, and
// truncate; the cut is relaxed until enough strings are found.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

#include "sub1_hip.h"

namespace {

constexpr int kCount = SUB1_DICT_ENTRIES;
constexpr int kMaxPairs = 14;  // sub1.py:54

struct Str {
  double key;
  uint8_t len;
  uint8_t s[kMaxPairs];
};

inline bool str_less(const Str &a, const Str &b) {
  if (a.key != b.key) return a.key < b.key;
  int n = std::min<int>(a.len, b.len);
  int c = std::memcmp(a.s, b.s, n);
  if (c != 0) return c < 0;
  return a.len < b.len;
}

void enumerate(const double q[9], double cut, const Str &parent, std::vector<Str> &out) {
  if (parent.len == kMaxPairs) return;
  for (int i = 0; i < 9; i++) {
    double k = parent.key * q[i];
    if (k > cut) continue;  // keys only move towards zero along a string
    Str ch = parent;
    ch.key = k;
    ch.s[ch.len++] = static_cast<uint8_t>(i);
    out.push_back(ch);
    enumerate(q, cut, ch, out);
  }
}

}  // namespace

namespace sub1 {

// Dictionary strings in index order.  Returns false if something is off.
bool dictionary_strings(std::vector<Str> &res) {
  // sub1.py:33-44: p = [.885, (1-.885)/2, (1-.885)/2]; q[3a+b] = (1.0*p[a])*p[b]
  const double zeros = .885;
  const double p[3] = {zeros, (1 - zeros) / 2, (1 - zeros) / 2};
  double q[9];
  for (int a = 0; a < 3; a++)
    for (int b = 0; b < 3; b++) q[3 * a + b] = (1. * p[a]) * p[b];

  Str root;
  std::memset(&root, 0, sizeof root);
  root.key = -1.;
  double cut = -1e-5;
  for (int attempt = 0; attempt < 40; attempt++) {
    res.clear();
    enumerate(q, cut, root, res);
    if (static_cast<int>(res.size()) >= kCount) break;
    cut /= 4;
  }
  if (static_cast<int>(res.size()) < kCount) return false;
  std::sort(res.begin(), res.end(), str_less);
  res.resize(kCount);
  return true;
}

}  // namespace sub1

extern "C" int sub1_build_tables(int32_t *dec_host, int32_t *trie_host) {
  std::vector<Str> res;
  if (!sub1::dictionary_strings(res)) return SUB1_ERR_INTERNAL;

  if (dec_host) {
    // sub1.py:60-72: pairs 0-6 in word 2i, pairs 7-13 in word 2i+1; pair j of
    // a word at bits 4+4j (even-position weight in the low two bits); the low
    // nibble of both words is the pair count.
    for (int i = 0; i < kCount; i++) {
      uint32_t w[2] = {0u, 0u};
      for (int j = 0; j < res[i].len; j++) {
        uint32_t r = res[i].s[j];
        uint32_t nib = (r % 3) | ((r / 3) << 2);
        w[j / 7] |= nib << (4 * (j % 7));
      }
      dec_host[2 * i] = static_cast<int32_t>((w[0] << 4) | res[i].len);
      dec_host[2 * i + 1] = static_cast<int32_t>((w[1] << 4) | res[i].len);
    }
  }

  if (trie_host) {
    // sub1.py:74-97: row = node, column = pair symbol, value = child entry or
    // -1; the root is row 65536.  A string's parent precedes it in the order.
    std::fill(trie_host, trie_host + SUB1_TRIE_WORDS, -1);
    for (int i = 0; i < kCount; i++) {
      int node = kCount;
      for (int j = 0; j + 1 < res[i].len; j++) {
        node = trie_host[9 * node + res[i].s[j]];
        if (node < 0) return SUB1_ERR_INTERNAL;
      }
      trie_host[9 * node + res[i].s[res[i].len - 1]] = i;
    }
  }
  return SUB1_OK;
}

// ---------------------------------------------------------------------------
// Kernel tables: a renumbering of the dictionary under which the decode table
// fits LDS.
//
// An entry has at most three non-zero weights.  Entries that differ only in
// the symbols (row min / row max) of their non-zeros form a group; 7164 groups
// of three non-zeros are complete (all 8 symbol patterns are entries).  The
// kernels work on streams whose codes were renumbered so that
//   * a complete group g owns the 8 consecutive codes B + 8g .. B + 8g + 7 and
//     the code's low three bits ARE the symbol pattern (bit j set = non-zero j
//     is the row max): the group needs ONE table word;
//   * every other entry (B of them) owns one code below B and one table word
//     of its own, and its code is chosen so that its low three bits agree
//     with its symbols too (bits of empty slots are free).  This is what lets
//     the kernel insert the code's low bits into the table word unconditionally.
// Table word: bytes 0, 1 and 3 = slots 0, 1 and 2, each the dword offset of a
// non-zero in the activation array relative to the codeword's first column,
// with the symbol bit cleared; byte 2 = 6 * pair count.  The activation array
// spends 6 dwords per column pair: [A_even, B_even, A_odd, B_odd, 0, 0], A =
// value routed to the row-min sum, B = to the row-max sum, so a non-zero at
// in-code position p = 2m + q with symbol s sits at 6m + 2q + (s - 1).
// Non-zeros fill the slots from slot 0; an empty slot 0 or 1 points at the zero
// dwords of its own pair (offset 4).  Half of all codewords in a stream leave
// slot 2 empty: such a word carries 0x82 there, bit 7 (the word's sign bit)
// telling the kernel to drop the column from the address, so that all those
// lanes read ONE dword (130, a zero of pair 21) and take no extra LDS bank.
//
// Slots are in column order, except that slots feeding different sums may be
// swapped (that changes no sum's order of additions): the freedom is needed to
// balance the code classes.
namespace {

struct Parsed {
  int len;        // pairs
  int n;          // non-zeros
  int pos[3];
  int sym[3];     // 1 or 2
};

bool parse_entry(const Str &s, Parsed &p) {
  p.len = s.len;
  p.n = 0;
  for (int j = 0; j < s.len; j++) {
    int r = s.s[j];
    int d[2] = {r % 3, r / 3};
    for (int q = 0; q < 2; q++) {
      if (!d[q]) continue;
      if (p.n == 3) return false;
      p.pos[p.n] = 2 * j + q;
      p.sym[p.n] = d[q];
      p.n++;
    }
  }
  return true;
}

inline uint32_t slot_offset(int pos) { return 6u * (pos / 2) + 2u * (pos & 1); }
constexpr uint32_t kEmptySlot = 4;
constexpr uint32_t kEmptyLastSlot = 0x82;   // bit 7: empty; 128 + 2 = zero dword of pair 21

struct Arrangement {
  int cls_mask;   // bits of the code class that are fixed
  int cls_val;    // their values
  int slot_of[3]; // slot index of non-zero i
};

// All ways to put the non-zeros of an entry into the three slots such that
// non-zeros with the same symbol stay in column order.
void arrangements(const Parsed &p, std::vector<Arrangement> &out) {
  out.clear();
  int perm[3] = {0, 1, 2};
  do {
    // perm[i] = slot of non-zero i (only the first p.n matter)
    bool ok = true;
    for (int a = 0; a < p.n && ok; a++) {
      if (perm[a] >= p.n) ok = false;   // empty slots come last
      for (int b = a + 1; b < p.n && ok; b++)
        if (p.sym[a] == p.sym[b] && perm[a] > perm[b]) ok = false;
    }
    if (!ok) continue;
    Arrangement ar;
    ar.cls_mask = 0;
    ar.cls_val = 0;
    for (int i = 0; i < 3; i++) ar.slot_of[i] = perm[i];
    for (int i = 0; i < p.n; i++) {
      ar.cls_mask |= 1 << perm[i];
      if (p.sym[i] == 2) ar.cls_val |= 1 << perm[i];
    }
    bool dup = false;
    for (const Arrangement &o : out)
      if (o.cls_mask == ar.cls_mask && o.cls_val == ar.cls_val) {
        bool same = true;
        for (int i = 0; i < p.n; i++) same = same && o.slot_of[i] == ar.slot_of[i];
        if (same) dup = true;
      }
    if (!dup) out.push_back(ar);
  } while (std::next_permutation(perm, perm + 3));
}

uint32_t table_word(const Parsed &p, const int slot_of[3]) {
  uint32_t f[3] = {kEmptySlot, kEmptySlot, kEmptyLastSlot};
  for (int i = 0; i < p.n; i++) f[slot_of[i]] = slot_offset(p.pos[i]);
  return f[0] | (f[1] << 8) | (static_cast<uint32_t>(6 * p.len) << 16) | (f[2] << 24);
}

}  // namespace

extern "C" int sub1_build_kernel_tables(uint16_t *recode_host, uint32_t *table_host,
                                        int32_t *single_codes, int32_t *table_words) {
  std::vector<Str> res;
  if (!sub1::dictionary_strings(res)) return SUB1_ERR_INTERNAL;
  std::vector<Parsed> ps(kCount);
  for (int i = 0; i < kCount; i++)
    if (!parse_entry(res[i], ps[i])) return SUB1_ERR_INTERNAL;

  // groups of three non-zeros keyed by (length, positions)
  struct Group {
    int member[8];
    int count;
  };
  std::vector<Group> groups;
  std::vector<int> group_of(kCount, -1);
  {
    std::vector<std::pair<uint32_t, int>> keyed;
    for (int i = 0; i < kCount; i++)
      if (ps[i].n == 3) {
        uint32_t key = (ps[i].len << 15) | (ps[i].pos[0] << 10) | (ps[i].pos[1] << 5) | ps[i].pos[2];
        keyed.push_back({key, i});
      }
    std::sort(keyed.begin(), keyed.end());
    for (size_t a = 0; a < keyed.size();) {
      size_t b = a;
      Group g;
      g.count = 0;
      for (int k = 0; k < 8; k++) g.member[k] = -1;
      while (b < keyed.size() && keyed[b].first == keyed[a].first) {
        const Parsed &p = ps[keyed[b].second];
        int pat = (p.sym[0] == 2) | ((p.sym[1] == 2) << 1) | ((p.sym[2] == 2) << 2);
        g.member[pat] = keyed[b].second;
        g.count++;
        b++;
      }
      if (g.count == 8) {
        for (int k = 0; k < 8; k++) group_of[g.member[k]] = static_cast<int>(groups.size());
        groups.push_back(g);
      }
      a = b;
    }
  }
  // complete groups in order of their first entry, so the numbering is canonical
  std::sort(groups.begin(), groups.end(), [](const Group &a, const Group &b) {
    return *std::min_element(a.member, a.member + 8) < *std::min_element(b.member, b.member + 8);
  });

  std::vector<int> singles;
  for (int i = 0; i < kCount; i++)
    if (group_of[i] < 0) singles.push_back(i);
  const int nb = static_cast<int>(singles.size());
  if (nb % 8 != 0 || nb + 8 * static_cast<int>(groups.size()) != kCount) return SUB1_ERR_INTERNAL;
  const int words = nb + static_cast<int>(groups.size());
  if (single_codes) *single_codes = nb;
  if (table_words) *table_words = words;
  if (!recode_host && !table_host) return SUB1_OK;

  std::vector<uint16_t> recode(kCount);
  std::vector<uint32_t> table(words);

  // Singles: every code class (the code's low three bits) takes exactly nb / 8
  // of them, and an entry fits a class if one of its arrangements agrees with
  // the class's bits.  Entries with the same set of admissible classes are
  // interchangeable, so the assignment is a small transportation problem
  // (sets of classes x 8 classes), solved by augmenting paths; within a set the
  // entries go to their classes in dictionary order, which makes the numbering
  // canonical.
  std::vector<std::vector<Arrangement>> opts(nb);
  std::vector<int> admissible(nb, 0);
  for (int k = 0; k < nb; k++) {
    arrangements(ps[singles[k]], opts[k]);
    for (const Arrangement &a : opts[k])
      for (int c = 0; c < 8; c++)
        if ((c & a.cls_mask) == a.cls_val) admissible[k] |= 1 << c;
  }
  const int cap = nb / 8;
  int supply[256] = {0};
  for (int k = 0; k < nb; k++) supply[admissible[k]]++;
  static int flow[256][8];
  int load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int m = 0; m < 256; m++)
    for (int c = 0; c < 8; c++) flow[m][c] = 0;
  for (int m = 1; m < 256; m++) {
    while (supply[m] > 0) {
      // breadth-first search from set m for a class with room, moving units
      // between classes through the sets that hold them
      int from_set[8], via_class[8];
      bool seen[8] = {false, false, false, false, false, false, false, false};
      int queue[8], head = 0, tail = 0, found = -1;
      for (int c = 0; c < 8; c++)
        if (m >> c & 1) {
          seen[c] = true;
          from_set[c] = m;
          via_class[c] = -1;
          queue[tail++] = c;
        }
      while (head < tail && found < 0) {
        const int c = queue[head++];
        if (load[c] < cap) {
          found = c;
          break;
        }
        // class c is full: one of its units, from set t, may move to class d
        for (int t = 1; t < 256; t++) {
          if (!flow[t][c]) continue;
          for (int d = 0; d < 8; d++)
            if ((t >> d & 1) && !seen[d]) {
              seen[d] = true;
              from_set[d] = t;
              via_class[d] = c;
              queue[tail++] = d;
            }
        }
      }
      if (found < 0) return SUB1_ERR_INTERNAL;  // classes cannot be balanced
      // push one unit along the path
      int d = found;
      load[d]++;
      while (via_class[d] >= 0) {
        const int t = from_set[d], c = via_class[d];
        flow[t][d]++;
        flow[t][c]--;
        d = c;
      }
      flow[m][d]++;
      supply[m]--;
    }
  }
  int used[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k = 0; k < nb; k++) {
    const int m = admissible[k];
    int c = 0;
    while (c < 8 && !flow[m][c]) c++;
    if (c == 8) return SUB1_ERR_INTERNAL;
    flow[m][c]--;
    const Arrangement *chosen = nullptr;
    for (const Arrangement &a : opts[k])
      if ((c & a.cls_mask) == a.cls_val) {
        chosen = &a;
        break;
      }
    if (!chosen) return SUB1_ERR_INTERNAL;
    const int code = c + 8 * used[c]++;
    recode[singles[k]] = static_cast<uint16_t>(code);
    table[code] = table_word(ps[singles[k]], chosen->slot_of);
  }

  const int identity[3] = {0, 1, 2};
  for (size_t g = 0; g < groups.size(); g++) {
    for (int pat = 0; pat < 8; pat++)
      recode[groups[g].member[pat]] = static_cast<uint16_t>(nb + 8 * g + pat);
    table[nb + g] = table_word(ps[groups[g].member[0]], identity);
  }

  if (recode_host) std::copy(recode.begin(), recode.end(), recode_host);
  if (table_host) std::copy(table.begin(), table.end(), table_host);
  return SUB1_OK;
}
