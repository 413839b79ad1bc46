"""Writes the golden vectors of this directory (inputs and expected outputs, as .npz).

The reference's tests for this path store no vectors (they draw random data and compare with torch
at run time), so the expected outputs here come from what the reference's tests compare against,
evaluated on the CPU with library routines only -- torch's fp8 / bf16 casts, IEEE fp32 arithmetic,
float64 matmul, exact rational sums -- and never from this repository's oracle or kernels:

    fp8_cast.npz        torch CPU `.to(torch.float8_e4m3fn)` on every rounding boundary of the format
    quant_1x128.npz     pertoken_quant on [-1, G] views (aiter/ops/quant.py:64-94, :331-346)
    weight_128x128.npz  the same on 128x128 blocks (op_tests/multigpu_tests/test_dispatch_combine.py:180-204)
    gemm_blockscale.npz run_torch of op_tests/test_gemm_a8w8_blockscale.py:28-54, in float64 and in fp32
    rmsnorm_quant.npz   F.rms_norm (op_tests/test_rmsnorm2dFusedAddQuant.py:23-55) and the same formula
                        with an exactly rounded mean of squares, then the 1x128 quant
    moe_routing.npz     softmax + top-k and the sorted layout of op_tests/test_moe_sorting.py:44-105,
                        by plain loops
    moe_layer.npz       torch_moe_blockscale of op_tests/test_moe_blockscale.py:19-101 by per-token loops
                        in float64

Run from the repository root:  python tests/golden/make_fixtures.py
The tests that read these files are tests/test_golden.py (CPU: the oracle) and
tests/test_golden_gpu.py (the library, through its entry points).
"""

import os
from fractions import Fraction

import numpy as np
import torch
import torch.nn.functional as F

OUT = os.path.dirname(os.path.abspath(__file__))
FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


def bits32(t):
    return t.contiguous().view(torch.int32).numpy().view(np.uint32).copy()


def codes16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def codes8(t):
    return t.contiguous().view(torch.uint8).numpy().copy()


def save(name, **arrays):
    path = os.path.join(OUT, name)
    np.savez_compressed(path, **arrays)
    print(f"{name}: {os.path.getsize(path)} bytes, " + ", ".join(f"{k}{list(v.shape)}" for k, v in arrays.items()))


# ---------------------------------------------------------------- fp32 -> e4m3fn
def e4m3_values():
    """The 127 non-negative finite values of OCP e4m3fn (bias 7, no infinities), by the format's formula."""
    vals = []
    for code in range(0x7F):
        e, m = code >> 3, code & 7
        vals.append(m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
    return np.array(vals, dtype=np.float64)


def make_fp8_cast():
    v = e4m3_values()
    mids = (v[:-1] + v[1:]) / 2  # exactly representable in fp32
    pts = np.concatenate([v, mids, [464.0, 465.0, 480.0, 1e30, 2.0 ** -10, 2.0 ** -11, 1e-30, 1e-45]]).astype(np.float32)
    around = np.concatenate([pts, np.nextafter(pts, np.float32(np.inf)), np.nextafter(pts, np.float32(-np.inf))])
    rng = np.random.default_rng(0)
    rand = (rng.standard_normal(4096) * 10.0 ** rng.uniform(-4, 3, 4096)).astype(np.float32)
    x = np.concatenate([around, -around, rand, np.array([np.inf, -np.inf, np.nan, 0.0, -0.0], dtype=np.float32)])
    t = torch.from_numpy(x.copy())
    save("fp8_cast.npz", f32_bits=bits32(t), codes=codes8(t.to(FP8)))


# ---------------------------------------------------------------- 1 x G group quant
def pertoken_quant(x2d):
    """aiter/ops/quant.py:64-94 on rows of x2d (float32): scale = amax / 448 (0 -> 1), y = (x / scale) as fp8."""
    amax = x2d.abs().amax(dim=-1, keepdim=True)
    scale = amax / FP8_MAX
    scale[scale == 0] = 1
    return (x2d / scale).to(FP8), scale.view(-1)


def make_quant():
    torch.manual_seed(0)
    x = torch.randn(32, 1024).bfloat16()  # the reference's own small case
    special = torch.zeros(8, 1024)
    special[1, :] = 448.0
    special[2, ::7] = -3.0
    special[2, 5] = 150.0  # one outlier per group region
    special[3] = torch.randn(1024) * 1e-30
    special[4] = torch.randn(1024) * 1e30
    special[5] = torch.randn(1024)
    special[5, 100] = float("inf")
    special[5, 700] = float("nan")
    special[6] = torch.linspace(-500, 500, 1024)
    special[7, 3] = -0.0
    special[7, 130] = 2.0 ** -126
    x = torch.cat([x, special.bfloat16()])
    y, s = pertoken_quant(x.float().view(-1, 128))
    x16 = (torch.randn(4, 256) * 3).half()
    y16, s16 = pertoken_quant(x16.float().view(-1, 64))
    save("quant_1x128.npz", x_bf16=codes16(x), y=codes8(y.view(x.shape)), scale_bits=bits32(s).reshape(x.shape[0], -1),
         x_fp16=codes16(x16), y_fp16_g64=codes8(y16.view(x16.shape)), scale_fp16_g64_bits=bits32(s16).reshape(4, -1))


# ---------------------------------------------------------------- 128 x 128 weight quant
def weight_quant(w):
    """[N, K] -> fp8 codes and [ceil(N/128), K/128] scales: each 128x128 block is one pertoken_quant row."""
    n, k = w.shape
    nb, kb = (n + 127) // 128, k // 128
    padded = torch.zeros(nb * 128, k)
    padded[:n] = w.float()
    blocks = padded.view(nb, 128, kb, 128).permute(0, 2, 1, 3).reshape(nb * kb, 128 * 128)
    q, s = pertoken_quant(blocks)
    q = q.view(torch.uint8).view(nb, kb, 128, 128).permute(0, 2, 1, 3).reshape(nb * 128, k)[:n]
    return q.view(FP8), s.view(nb, kb)


def make_weight_quant():
    torch.manual_seed(1)
    w = (torch.randn(192, 256) * 0.02).bfloat16()  # the second row block has 64 rows
    w[130, 140:150] = 0.7
    q, s = weight_quant(w)
    save("weight_128x128.npz", w_bf16=codes16(w), q=codes8(q), scale_bits=bits32(s))


# ---------------------------------------------------------------- block-scale GEMM
def make_gemm():
    torch.manual_seed(2)
    m, n, k = 5, 192, 384
    x = torch.randn(m, k).bfloat16()
    xq, xs = pertoken_quant(x.float().view(-1, 128))
    xq, xs = xq.view(m, k), xs.view(m, k // 128)
    wq, ws = weight_quant((torch.randn(n, k) * 0.02).bfloat16())
    xd = xq.double().view(m, k // 128, 128) * xs.double().unsqueeze(-1)
    wsd = ws.double().repeat_interleave(128, 0)[:n].repeat_interleave(128, 1)
    wd = wq.double() * wsd
    out64 = xd.view(m, k) @ wd.t()
    out32 = F.linear(xd.view(m, k).float(), wd.float()).bfloat16()
    save("gemm_blockscale.npz", xq=codes8(xq), wq=codes8(wq), x_scale_bits=bits32(xs), w_scale_bits=bits32(ws),
         out_f64=out64.numpy(), out_bf16=codes16(out32))


# ---------------------------------------------------------------- RMSNorm (+ residual) + quant
def rne32(fr):
    """Fraction -> nearest float32 (ties to even); exact for the magnitudes used here."""
    c = np.float32(float(fr))
    lo, hi = np.nextafter(c, np.float32(-np.inf)), np.nextafter(c, np.float32(np.inf))
    best = min((abs(Fraction(float(v)) - fr), int(v.view(np.uint32)) & 1, v) for v in (lo, c, hi))
    return best[2]


def rmsnorm_exact(x, w, eps):
    """bf16(RN32(x * rstd) * w) with rstd = 1 / sqrt(RN32(mean of squares) + eps) in fp32; the mean is the
    correctly rounded one (exact rational sum)."""
    rows, hidden = x.shape
    xf, wf = x.float().numpy(), w.float().numpy()
    out = np.empty((rows, hidden), dtype=np.float32)
    for r in range(rows):
        total = sum(Fraction(float(v)) ** 2 for v in xf[r])
        mean = rne32(total / hidden)
        rstd = np.float32(1.0) / np.sqrt(np.float32(mean + np.float32(eps)))
        out[r] = (xf[r] * rstd).astype(np.float32) * wf
    return torch.from_numpy(out).bfloat16()


def make_rmsnorm():
    torch.manual_seed(3)
    rows, hidden, eps = 6, 512, 1e-6
    x = (torch.randn(rows, hidden) * torch.tensor([1.0, 0.01, 30.0, 1.0, 1e-3, 5.0]).view(-1, 1)).bfloat16()
    res = torch.randn(rows, hidden).bfloat16()
    w = (torch.rand(hidden) + 0.5).bfloat16()
    lib = F.rms_norm(x, (hidden,), weight=w, eps=eps)
    exact = rmsnorm_exact(x, w, eps)
    y, s = pertoken_quant(exact.float().view(-1, 128))
    summed = x + res  # rounded to bf16, as the reference's test does before norming
    exact_add = rmsnorm_exact(summed, w, eps)
    ya, sa = pertoken_quant(exact_add.float().view(-1, 128))
    save("rmsnorm_quant.npz", x=codes16(x), residual=codes16(res), weight=codes16(w), eps=np.float32(eps),
         out_torch=codes16(lib), out_exact=codes16(exact), y=codes8(y.view(rows, hidden)),
         scale_bits=bits32(s).reshape(rows, -1), residual_out=codes16(summed), out_add_exact=codes16(exact_add),
         y_add=codes8(ya.view(rows, hidden)), scale_add_bits=bits32(sa).reshape(rows, -1))


# ---------------------------------------------------------------- MoE routing and sorting
def sort_by_loops(ids, weights, experts, block, mask=None):
    """Sorted layout of op_tests/test_moe_sorting.py:44-105: per (local) expert its (token, slot) pairs in
    (token, slot) order as slot << 24 | token, padded to a multiple of `block` with topk << 24 | tokens."""
    tokens, topk = ids.shape
    local, nxt = {}, 0
    for e in range(experts):
        if mask is None or mask[e]:
            local[e] = nxt
            nxt += 1
    s_ids, s_w, s_e = [], [], []
    pad = (topk << 24) | tokens
    for e in range(experts):
        if e not in local:
            continue
        pairs = [(t, k) for t in range(tokens) for k in range(topk) if ids[t, k] == e]
        if not pairs:
            continue
        for t, k in pairs:
            s_ids.append((k << 24) | t)
            s_w.append(weights[t, k])
        while len(s_ids) % block:
            s_ids.append(pad)
            s_w.append(0.0)
        s_e += [local[e]] * ((len(pairs) + block - 1) // block)
    return np.array(s_ids, dtype=np.int32), np.array(s_w, dtype=np.float32), np.array(s_e, dtype=np.int32)


def make_moe_routing():
    torch.manual_seed(4)
    tokens, experts, topk, block = 11, 6, 3, 4
    gating = torch.randn(tokens, experts)
    gating[2, 1] = gating[2, 4]  # a tie: the lower index wins
    prob = torch.softmax(gating.double(), dim=-1)
    ids = np.zeros((tokens, topk), dtype=np.int32)
    wts = np.zeros((tokens, topk), dtype=np.float64)
    for t in range(tokens):
        order = sorted(range(experts), key=lambda e: (-prob[t, e].item(), e))[:topk]
        ids[t] = order
        wts[t] = [prob[t, e].item() for e in order]
    renorm = (wts / wts.sum(-1, keepdims=True)).astype(np.float32)
    s_ids, s_w, s_e = sort_by_loops(ids, renorm, experts, block)
    mask = np.array([1, 0, 1, 1, 0, 1], dtype=np.int32)
    m_ids, m_w, m_e = sort_by_loops(ids, renorm, experts, block, mask)
    save("moe_routing.npz", gating=gating.numpy(), topk_ids=ids, topk_weights=wts.astype(np.float32),
         topk_weights_renorm=renorm, block=np.int32(block), sorted_ids=s_ids, sorted_weights=s_w, sorted_expert_ids=s_e,
         expert_mask=mask, masked_sorted_ids=m_ids, masked_sorted_weights=m_w, masked_sorted_expert_ids=m_e)


# ---------------------------------------------------------------- MoE layer
def make_moe_layer():
    torch.manual_seed(5)
    tokens, dim, inter, experts, topk = 5, 256, 128, 4, 2
    x = torch.randn(tokens, dim).bfloat16()
    xq, xs = pertoken_quant(x.float().view(-1, 128))
    xq, xs = xq.view(tokens, dim), xs.view(tokens, dim // 128)
    w1q, w1s = weight_quant((torch.randn(experts * 2 * inter, dim) * 0.1).bfloat16())
    w2q, w2s = weight_quant((torch.randn(experts * dim, inter) * 0.1).bfloat16())
    ids = np.array([[0, 2], [3, 1], [2, 0], [1, 3], [0, 1]], dtype=np.int32)
    wts = torch.softmax(torch.randn(tokens, topk), -1).numpy().astype(np.float32)

    def dequant_w(q, s, e, rows, k):
        qq = q.double().view(experts, rows, k)[e]
        ss = s.double().view(experts, rows // 128, k // 128)[e].repeat_interleave(128, 0).repeat_interleave(128, 1)
        return qq * ss

    xd = (xq.double().view(tokens, dim // 128, 128) * xs.double().unsqueeze(-1)).view(tokens, dim)
    out = torch.zeros(tokens, dim, dtype=torch.float64)
    out_q = torch.zeros(tokens, dim, dtype=torch.float64)  # with the fp8 rounding of the activation product
    for t in range(tokens):
        for k in range(topk):
            e = int(ids[t, k])
            h = dequant_w(w1q, w1s, e, 2 * inter, dim) @ xd[t]
            act = F.silu(h[:inter]) * h[inter:]
            w2 = dequant_w(w2q, w2s, e, dim, inter)
            out[t] += float(wts[t, k]) * (w2 @ act)
            aq, asc = pertoken_quant(act.float().bfloat16().float().view(-1, 128))
            act_q = (aq.double().view(-1, 128) * asc.double().view(-1, 1)).view(-1)
            out_q[t] += float(wts[t, k]) * (w2 @ act_q)
    save("moe_layer.npz", xq=codes8(xq), x_scale_bits=bits32(xs), w1q=codes8(w1q).reshape(experts, 2 * inter, dim),
         w1_scale_bits=bits32(w1s).reshape(experts, -1), w2q=codes8(w2q).reshape(experts, dim, inter),
         w2_scale_bits=bits32(w2s).reshape(experts, -1), topk_ids=ids, topk_weights=wts, out_f64=out.numpy(),
         out_f64_fp8_product=out_q.numpy())


if __name__ == "__main__":
    torch.set_num_threads(1)
    make_fp8_cast()
    make_quant()
    make_weight_quant()
    make_gemm()
    make_rmsnorm()
    make_moe_routing()
    make_moe_layer()
