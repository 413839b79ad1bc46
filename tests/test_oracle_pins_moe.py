"""Pins for the mixture-of-experts restatements in oracle/torch_ref.py (CPU only).

The reference holds no stored vectors for this path (its tests draw random data), so each
function is pinned by an independent formulation on small inputs and by what the definition fixes:
brute force over (token, slot) pairs for the sorted layout, torch.topk and a tie known answer for
the routing, a per-token dense fp64 evaluation built on the (separately pinned) block-scale GEMM
oracle for the experts."""

import torch
import torch.nn.functional as F

from oracle import torch_ref as tr


def brute_force_sorting(ids, w, experts, block, mask=None, local_tokens=None):
    m, topk = ids.shape
    rows = m if local_tokens is None else local_tokens
    pad = (topk << 24) | m
    out_ids, out_w, out_e = [], [], []
    skipped = 0
    for e in range(experts):
        if mask is not None and mask[e] == 0:
            skipped += 1
            continue
        pairs = [(t, k) for t in range(rows) for k in range(topk) if int(ids[t, k]) == e]
        for (t, k) in pairs:
            out_ids.append((k << 24) | t)
            out_w.append(float(w[t, k]))
        fill = (-len(pairs)) % block
        out_ids += [pad] * fill
        out_w += [None] * fill
        out_e += [e - skipped] * ((len(pairs) + block - 1) // block)
    return out_ids, out_w, out_e


def test_moe_sorting_ref_against_brute_force():
    g = torch.Generator().manual_seed(0)
    for (m, experts, topk, block) in [(1, 4, 2, 4), (9, 5, 3, 2), (40, 8, 2, 32), (17, 3, 1, 8), (6, 16, 4, 1)]:
        ids = torch.stack([torch.randperm(experts, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
        w = torch.rand(m, topk, generator=g)
        for mask, local in [(None, None), (torch.tensor([1, 0] * 8)[:experts].int(), None), (None, m // 2)]:
            s_ids, s_w, s_e, post = tr.moe_sorting_ref(ids, w, experts, block, mask, local)
            b_ids, b_w, b_e = brute_force_sorting(ids, w, experts, block, mask, local)
            n = len(b_ids)
            assert post.tolist() == [n, m if local is None else local]
            assert s_ids[:n].tolist() == b_ids
            assert (s_ids[n:] == ((topk << 24) | m)).all()
            assert s_e[: len(b_e)].tolist() == b_e and (s_e[len(b_e):] == -1).all()
            for i, v in enumerate(b_w):
                if v is not None:
                    assert s_w[i].item() == torch.tensor(v, dtype=torch.float32).item()
            # sizes the reference allocates (aiter/fused_moe.py:209-215)
            assert s_ids.numel() == m * topk + experts * block - topk
            assert s_e.numel() == (s_ids.numel() + block - 1) // block


def test_moe_sorting_ref_invariants():
    g = torch.Generator().manual_seed(1)
    m, experts, topk, block = 300, 32, 6, 32
    ids = torch.stack([torch.randperm(experts, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    w = torch.rand(m, topk, generator=g)
    s_ids, s_w, s_e, post = tr.moe_sorting_ref(ids, w, experts, block)
    n = int(post[0])
    assert n % block == 0
    real = s_ids[:n][(s_ids[:n] & 0xFFFFFF) < m]
    # every routed pair exactly once
    keys = ((real & 0xFFFFFF).long() * topk + (real >> 24).long()).sort().values
    assert torch.equal(keys, torch.arange(m * topk))
    # blocks are homogeneous and experts ascend; pairs ascend inside an expert
    for b in range(n // block):
        blk = s_ids[b * block:(b + 1) * block]
        e = int(s_e[b])
        for v in blk.tolist():
            if (v & 0xFFFFFF) < m:
                assert int(ids[v & 0xFFFFFF, v >> 24]) == e
    assert (s_e[: n // block][1:] >= s_e[: n // block][:-1]).all()


def test_fused_topk_ref_against_torch_topk_and_ties():
    g = torch.Generator().manual_seed(2)
    gating = torch.randn(50, 64, generator=g)
    for renorm in (True, False):
        w, ids = tr.fused_topk_ref(gating, 6, renorm)
        pv, pi = torch.topk(torch.softmax(gating, -1), 6, dim=-1)
        assert torch.equal(ids.long(), pi)
        expect = pv / pv.sum(-1, keepdim=True) if renorm else pv
        assert torch.allclose(w, expect, rtol=1e-6)
        if renorm:
            assert torch.allclose(w.sum(-1), torch.ones(50), atol=1e-6)
    tie = torch.zeros(2, 8)
    tie[1, 5] = 1.0
    w, ids = tr.fused_topk_ref(tie, 3, False)
    assert ids.tolist() == [[0, 1, 2], [5, 0, 1]]
    assert torch.allclose(w[0], torch.full((3,), 1 / 8))


def dense_token_eval(p, t, activation, compute=torch.float64):
    """out[t] = sum_k w_k * W2_e (act(W1g_e x) * (W1u_e x)), every matrix dequantised through the
    block-scale GEMM oracle's dequantiser."""
    dim = p["aq"].shape[1]
    inter = p["w2q"].shape[2]
    acc = torch.zeros(dim, dtype=compute)
    for k in range(p["ti"].shape[1]):
        e = int(p["ti"][t, k])
        s1 = p["w1s"][e].view(2 * inter // 128, dim // 128)
        s2 = p["w2s"][e].view(dim // 128, inter // 128)
        x, w1 = tr.dequant_blockscale(p["aq"][t:t + 1], p["w1q"][e], p["asc"][t:t + 1], s1)
        h = (x.to(compute) @ w1.to(compute).t())[0]
        gate, up = h[:inter], h[inter:]
        act = (F.silu(gate) if activation == "silu" else F.gelu(gate)) * up
        ones = torch.ones(1, inter // 128)
        one_q = torch.ones(1, inter).to(tr.FP8)
        _, w2 = tr.dequant_blockscale(one_q, p["w2q"][e], ones, s2)
        acc += float(p["tw"][t, k]) * (w2.to(compute) @ act)
    return acc


def small_problem(seed, tokens=6, dim=256, inter=128, experts=4, topk=2):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, dim, generator=g).bfloat16()
    aq, asc = tr.per_1x128_quant(x)
    w1q, w1s, w2q, w2s = [], [], [], []
    for _ in range(experts):
        q, s = tr.weight_per_128x128_quant((torch.randn(2 * inter, dim, generator=g) / 10).bfloat16())
        w1q.append(q), w1s.append(s.reshape(-1))
        q, s = tr.weight_per_128x128_quant((torch.randn(dim, inter, generator=g) / 10).bfloat16())
        w2q.append(q), w2s.append(s.reshape(-1))
    tw, ti = tr.fused_topk_ref(torch.randn(tokens, experts, generator=g), topk, True)
    return dict(aq=aq, asc=asc, w1q=torch.stack(w1q), w1s=torch.stack(w1s), w2q=torch.stack(w2q),
                w2s=torch.stack(w2s), tw=tw, ti=ti)


def test_moe_blockscale_ref_against_per_token_dense_evaluation():
    for activation in ("silu", "gelu"):
        p = small_problem(3)
        got = tr.moe_blockscale_ref(p["aq"], p["w1q"], p["w2q"], p["tw"], p["ti"], p["asc"], p["w1s"], p["w2s"],
                                    activation=activation, compute=torch.float64)
        for t in range(p["aq"].shape[0]):
            want = dense_token_eval(p, t, activation)
            # (the GEMM oracle's dequantiser multiplies code and scale in fp32)
            assert torch.allclose(got[t], want, rtol=1e-5, atol=1e-5), (activation, t)
        got32 = tr.moe_blockscale_ref(p["aq"], p["w1q"], p["w2q"], p["tw"], p["ti"], p["asc"], p["w1s"], p["w2s"],
                                      activation=activation)
        assert torch.allclose(got32.double(), got, rtol=1e-4, atol=1e-4)


def test_moe_blockscale_ref_single_expert_reduces_to_two_gemms():
    # one expert, top-1, weight 1: out = gemm(act(gemm(x, W1)), W2) with the pinned GEMM oracle
    p = small_problem(4, experts=1, topk=1)
    inter = p["w2q"].shape[2]
    dim = p["aq"].shape[1]
    h = tr.gemm_a8w8_blockscale_ref_f64(p["aq"], p["w1q"][0], p["asc"], p["w1s"][0].view(2 * inter // 128, dim // 128))
    act = F.silu(h[:, :inter]) * h[:, inter:]
    s2 = p["w2s"][0].view(dim // 128, inter // 128).double().repeat_interleave(128, 0).repeat_interleave(128, 1)
    want = act @ (p["w2q"][0].double() * s2).t()
    got = tr.moe_blockscale_ref(p["aq"], p["w1q"], p["w2q"], torch.ones_like(p["tw"]), p["ti"], p["asc"], p["w1s"],
                                p["w2s"], compute=torch.float64)
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)


def test_moe_blockscale_ref_expert_mask_and_a2_quant():
    p = small_problem(5, experts=4, topk=2)
    mask = torch.tensor([1, 0, 1, 1], dtype=torch.int32)
    keep = mask.bool()
    got = tr.moe_blockscale_ref(p["aq"], p["w1q"][keep], p["w2q"][keep], p["tw"], p["ti"], p["asc"], p["w1s"][keep],
                                p["w2s"][keep], expert_mask=mask, compute=torch.float64)
    # same as zeroing the routing weight of the pairs that point at expert 1
    tw = p["tw"].clone()
    tw[p["ti"] == 1] = 0
    want = tr.moe_blockscale_ref(p["aq"], p["w1q"], p["w2q"], tw, p["ti"], p["asc"], p["w1s"], p["w2s"],
                                 compute=torch.float64)
    assert torch.allclose(got, want, rtol=1e-9, atol=1e-9)
    # a2_quant: the activation product goes through bf16 and the (pinned) 1x128 quantiser; the result stays
    # within the fp8 rounding error of the unquantised one and is not identical to it
    plain = tr.moe_blockscale_ref(p["aq"], p["w1q"], p["w2q"], p["tw"], p["ti"], p["asc"], p["w1s"], p["w2s"])
    quant = tr.moe_blockscale_ref(p["aq"], p["w1q"], p["w2q"], p["tw"], p["ti"], p["asc"], p["w1s"], p["w2s"],
                                  a2_quant=True)
    rel = ((plain - quant).norm() / plain.norm()).item()
    assert 1e-3 < rel < 5e-2
