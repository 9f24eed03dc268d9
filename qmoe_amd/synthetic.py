"""Seeded synthetic ternary experts, generated and encoded on the GPU.

The benchmark configurations are too large to build through Python lists the
way reference test.py:146-161 does (Switch-c-2048 has 52 G weights per MoE
layer), so symbols are drawn with torch's seeded generator on the device and
encoded with the library's own pack kernels, several experts at a time as one
tall matrix (codes never span rows, so the per-expert streams are slices of
the tall stream).
"""
import torch

from . import sub1, sub1_hip

# Switch expert shapes (d_model, d_ff): reference test.py:139-143
SHAPES = {'base': (768, 3072), 'large': (1024, 4096), 'c2048': (2080, 6144)}


ROWS = 'rows'     # p_zero: the share of zeros differs from row to row (draw_symbols)


def draw_symbols(rows, width, p_zero, generator, device):
    """int32 [rows, width].  p_zero a number: iid, P(0)=p_zero,
    P(1)=P(2)=(1-p_zero)/2.  p_zero = ROWS: every row has its own share of
    zeros, uniform in 0.75..0.98, except that one row in a hundred is all zero
    and one in a hundred has no zero at all; within a row iid as above.  (What
    a quantiser leaves is not iid: the fixed dictionary and the row order of the
    prepared stream see rows of very different lengths.)"""
    u = torch.rand((rows, width), generator=generator, device=device)
    if p_zero == ROWS:
        kind = torch.rand(rows, generator=generator, device=device)
        share = 0.75 + 0.23 * torch.rand(rows, generator=generator, device=device)
        share = torch.where(kind < 0.01, torch.ones_like(share), share)
        share = torch.where(kind >= 0.99, torch.zeros_like(share), share)
        p = share[:, None]
    else:
        p = p_zero
    t = (u >= p).to(torch.int32)
    t += (u >= p + (1 - p) / 2).to(torch.int32)
    return t


def draw_minmax(rows, generator, device):
    """bf16 [2*rows]: (-s, +s) per row, s ~ U(0.01, 0.05)."""
    s = (0.01 + 0.04 * torch.rand(rows, generator=generator, device=device)).bfloat16()
    return torch.stack((-s, s), dim=1).flatten()


def pack_experts(experts, height, width, p_zero, generator, device, chunk_weights=1 << 28,
                 keep_symbols=False):
    """Encode `experts` matrices of [height, width].  Returns (list of w_comp
    chunks, row_off int32 [E, height+1] local to each expert, code counts int64
    [E] on the host, ter_minmax bf16 [E, 2*height], symbols or None)."""
    _, trie = sub1.device_tables(device)
    per = max(1, chunk_weights // (height * width))
    chunks, row_offs, counts, minmax, symbols = [], [], [], [], []
    for first in range(0, experts, per):
        n = min(per, experts - first)
        t = draw_symbols(n * height, width, p_zero, generator, device)
        if keep_symbols:
            symbols.append(t.to(torch.uint8).reshape(n, height, width))
        tall = torch.zeros(n * height + 1, dtype=torch.int32, device=device)
        chunks.append(sub1_hip.sub1pack(trie, t, tall))
        del t
        starts = tall[0:n * height:height]                        # [n]
        local = tall[:-1].reshape(n, height) - starts[:, None]
        ends = torch.cat((starts[1:], tall[-1:])) - starts
        row_offs.append(torch.cat((local, ends[:, None]), dim=1))
        counts.append(ends.to(torch.int64).cpu())
        minmax.append(draw_minmax(n * height, generator, device).reshape(n, 2 * height))
    return (chunks, torch.cat(row_offs).contiguous(), torch.cat(counts),
            torch.cat(minmax).contiguous(),
            torch.cat(symbols) if keep_symbols else None)


def build_stack(experts, d_model, d_ff, p_zero, seed, device='cuda:0', keep_symbols=False):
    """One MoE layer of seeded synthetic experts as an ExpertStack.  With
    keep_symbols also returns (wi symbols uint8 [E, d_ff, d_model], wo symbols
    uint8 [E, d_model, d_ff])."""
    device = torch.device(device)
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    dec, _ = sub1.device_tables(device)
    wi_chunks, wi_ro, wi_n, wi_mm, wi_sym = pack_experts(
        experts, d_ff, d_model, p_zero, g, device, keep_symbols=keep_symbols)
    wo_chunks, wo_ro, wo_n, wo_mm, wo_sym = pack_experts(
        experts, d_model, d_ff, p_zero, g, device, keep_symbols=keep_symbols)
    w_comp = torch.cat(wi_chunks + wo_chunks)
    del wi_chunks, wo_chunks
    bases = torch.zeros(2 * experts + 1, dtype=torch.int64)
    bases[1:] = torch.cat((wi_n, wo_n)).cumsum(0)
    stack = sub1_hip.ExpertStack(
        dec, w_comp, bases[:experts].to(device), bases[experts:2 * experts].to(device),
        wi_ro.flatten(), wo_ro.flatten(), wi_mm.flatten(), wo_mm.flatten(), d_model, d_ff)
    stack.wi_codes, stack.wo_codes = wi_n, wo_n          # host copies of the stream sizes
    stack.wi_base, stack.wo_base = bases[:experts], bases[experts:2 * experts]
    if keep_symbols:
        return stack, wi_sym, wo_sym
    return stack


def expert_layers(stack, e):
    """The (w_comp, row_off, ter_minmax) triples of expert e's wi and wo, as
    views into the stack: exactly the buffers a Sub1Linear would hold."""
    d_model, d_ff = stack.d_model, stack.d_ff
    wi = (stack.w_comp[int(stack.wi_base[e]):int(stack.wi_base[e]) + int(stack.wi_codes[e])],
          stack.wi_row_off.view(-1, d_ff + 1)[e], stack.wi_minmax.view(-1, 2 * d_ff)[e])
    wo = (stack.w_comp[int(stack.wo_base[e]):int(stack.wo_base[e]) + int(stack.wo_codes[e])],
          stack.wo_row_off.view(-1, d_model + 1)[e], stack.wo_minmax.view(-1, 2 * d_model)[e])
    return wi, wo


def activations(tokens, width, seed, device='cuda:0'):
    """x ~ N(0,1) rounded to bf16, [tokens, width]."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return torch.randn((tokens, width), generator=g, device=device).bfloat16()


def softmax_router(tokens, experts, seed, device='cuda:0'):
    """Top-1 expert per token from N(0,1) logits (softmax is monotone, so the
    argmax of the logits)."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    logits = torch.randn((tokens, experts), generator=g, device=device)
    return torch.softmax(logits, dim=-1).argmax(dim=-1).to(torch.int32)
