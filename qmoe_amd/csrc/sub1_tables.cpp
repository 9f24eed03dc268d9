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
