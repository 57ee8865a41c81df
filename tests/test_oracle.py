"""Pins the oracle (CPU only).

The reference holds no golden vectors for this path, so each form of the
oracle is checked against a library routine, against the other forms, against
closed forms of special cases and against invariants chosen so that a dropped
term, a wrong index (``//L`` vs ``%L``, ``<=`` vs ``<``), a wrong sign or a
transposed operand fails at least one check.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from cases import ORACLE_SMALL

D64 = torch.float64


def _inputs(B, T, H, D, L, G, mode, seed=0):
    return oracle.make_inputs(B, T, H, D, L, G, seed=seed, dtype=D64, depth_only=(mode == "depth_only"))


@pytest.mark.parametrize("case", ORACLE_SMALL)
def test_rows_equals_dense(case):
    B, T, H, D, L, G, mode, cb = case
    inp = _inputs(B, T, H, D, L, G, mode)
    o1, l1 = oracle.moda_rows(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], 0.37, G, mode, cb, dtype=D64)
    o2, l2 = oracle.moda_dense(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], 0.37, G, mode, cb, dtype=D64)
    assert torch.allclose(o1, o2, atol=1e-12, rtol=1e-10)
    assert torch.allclose(l1, l2, atol=1e-12, rtol=1e-10)


@pytest.mark.parametrize("case", ORACLE_SMALL)
def test_dense_equals_library_sdpa(case):
    """Form (ii) == torch's scaled_dot_product_attention with the same boolean mask."""
    B, T, H, D, L, G, mode, cb = case
    inp = _inputs(B, T, H, D, L, G, mode, seed=3)
    o, _ = oracle.moda_dense(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], 0.5, G, mode, cb, dtype=D64)
    mask = oracle.visible_mask(T, G, L, mode, cb)
    keys = [x for x in (inp["k"], inp["kd"]) if x is not None]
    vals = [x for x in (inp["v"], inp["vd"]) if x is not None]
    if mode == "depth_only":
        mask = mask[:, T:]
    kc = torch.cat(keys, 1).permute(0, 2, 1, 3)
    vc = torch.cat(vals, 1).permute(0, 2, 1, 3)
    ref = F.scaled_dot_product_attention(inp["q"].permute(0, 2, 1, 3), kc, vc, attn_mask=mask, scale=0.5)
    assert torch.allclose(o, ref.permute(0, 2, 1, 3), atol=1e-12, rtol=1e-10)


def test_visible_mask_brute_force():
    """Mask against a literal restatement of the visible set, element by element."""
    for (T, G, L, mode, cb) in [(7, 2, 3, "causal", 0), (7, 1, 2, "noncausal", 0), (9, 2, 3, "chunk_visible", 4),
                                (5, 4, 2, "depth_only", 0), (6, 1, 0, "causal", 0)]:
        m = oracle.visible_mask(T, G, L, mode, cb)
        for r in range(T * G):
            t = r // G
            for j in range(T):
                exp = {"causal": j <= t, "chunk_visible": j <= t, "noncausal": True, "depth_only": False}[mode]
                assert bool(m[r, j]) == exp
            for c in range(T * L):
                w = c // L
                if mode == "chunk_visible":
                    exp = (t // cb) * cb <= w <= t
                else:
                    exp = w == t
                assert bool(m[r, T + c]) == exp


def test_no_depth_is_textbook_causal_attention():
    inp = _inputs(2, 11, 3, 8, 0, 1, "causal", seed=5)
    o, lse = oracle.moda_dense(inp["q"], inp["k"], inp["v"], None, None, None, 1, "causal", dtype=D64)
    ref = F.scaled_dot_product_attention(inp["q"].permute(0, 2, 1, 3), inp["k"].permute(0, 2, 1, 3),
                                         inp["v"].permute(0, 2, 1, 3), is_causal=True)
    assert torch.allclose(o, ref.permute(0, 2, 1, 3), atol=1e-12)
    # lse is base 2: 2**lse == row sum of exp(logits)
    s = torch.einsum("bqhd,bkhd->bhqk", inp["q"], inp["k"]) / math.sqrt(8)
    s = s.masked_fill(~torch.ones(11, 11, dtype=torch.bool).tril(), float("-inf"))
    assert torch.allclose(torch.exp2(lse).permute(0, 2, 1), torch.exp(s).sum(-1), rtol=1e-10)


def test_single_token_is_softmax_over_one_plus_L():
    inp = _inputs(1, 1, 1, 8, 5, 1, "causal", seed=7)
    o, lse = oracle.moda_dense(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], 1.0, 1, "causal", dtype=D64)
    keys = torch.cat([inp["k"][0, :, 0], inp["kd"][0, :, 0]], 0)
    vals = torch.cat([inp["v"][0, :, 0], inp["vd"][0, :, 0]], 0)
    w = torch.softmax(keys @ inp["q"][0, 0, 0], 0)
    assert torch.allclose(o[0, 0, 0], w @ vals, atol=1e-12)


def test_replicated_depth_slots_closed_form():
    """kd, vd = L copies of (k_t, v_t)  ==  causal attention with log(1+L) added to the diagonal logit."""
    B, T, H, D, L = 1, 9, 2, 8, 3
    inp = _inputs(B, T, H, D, 0, 1, "causal", seed=11)
    kd = inp["k"].repeat_interleave(L, dim=1)
    vd = inp["v"].repeat_interleave(L, dim=1)
    o, lse = oracle.moda_dense(inp["q"], inp["k"], inp["v"], kd, vd, 0.3, 1, "causal", dtype=D64)
    s = torch.einsum("bqhd,bkhd->bhqk", inp["q"], inp["k"]) * 0.3
    s = s + torch.eye(T, dtype=D64) * math.log(1 + L)
    s = s.masked_fill(~torch.ones(T, T, dtype=torch.bool).tril(), float("-inf"))
    ref = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, -1), inp["v"])
    assert torch.allclose(o, ref, atol=1e-12)
    assert torch.allclose(lse.permute(0, 2, 1), torch.logsumexp(s, -1) / math.log(2), atol=1e-12)


def test_fda_equals_per_token_softmax():
    B, T, H, D, L, G = 2, 5, 2, 8, 4, 2
    inp = _inputs(B, T, H, D, L, G, "depth_only", seed=13)
    o, _ = oracle.moda_dense(inp["q"], None, None, inp["kd"], inp["vd"], 0.7, G, "depth_only", dtype=D64)
    q5 = inp["q"].view(B, T, G, H, D)
    kd5 = inp["kd"].view(B, T, L, H, D)
    vd5 = inp["vd"].view(B, T, L, H, D)
    w = torch.softmax(torch.einsum("btghd,btlhd->bthgl", q5, kd5) * 0.7, -1)
    ref = torch.einsum("bthgl,btlhd->btghd", w, vd5).reshape(B, T * G, H, D)
    assert torch.allclose(o, ref, atol=1e-12)


def test_chunk_visible_with_one_token_chunks_is_moda():
    inp = _inputs(1, 10, 2, 8, 3, 2, "causal", seed=17)
    a = oracle.moda_dense(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], None, 2, "chunk_visible", 1, dtype=D64)
    b = oracle.moda_dense(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], None, 2, "causal", dtype=D64)
    assert torch.allclose(a[0], b[0], atol=1e-13) and torch.allclose(a[1], b[1], atol=1e-13)


def test_constant_values_give_constant_output():
    inp = _inputs(1, 8, 2, 8, 3, 2, "causal", seed=19)
    v = torch.full_like(inp["v"], 2.5)
    vd = torch.full_like(inp["vd"], 2.5)
    o, _ = oracle.moda_dense(inp["q"], inp["k"], v, inp["kd"], vd, None, 2, "causal", dtype=D64)
    assert torch.allclose(o, torch.full_like(o, 2.5), atol=1e-12)


@pytest.mark.parametrize("case", ORACLE_SMALL)
def test_gradient_invariants(case):
    B, T, H, D, L, G, mode, cb = case
    inp = _inputs(B, T, H, D, L, G, mode, seed=23)
    r = oracle.moda_dense_fwd_bwd(inp, 0.41, G, mode, cb, dtype=D64)
    # sum_rows dV + sum_rows dVd == sum_rows dO   (softmax weights of a row sum to one)
    tot = torch.zeros(B, H, D, dtype=D64)
    for n in ("dv", "dvd"):
        if r[n] is not None:
            tot += r[n].sum(1)
    assert torch.allclose(tot, inp["do"].sum(1), atol=1e-10)
    # <q, dq> == <k, dk> + <kd, dkd>   (logits are bilinear in q and keys)
    lhs = (inp["q"] * r["dq"]).sum()
    rhs = sum((inp[n] * r["d" + n]).sum() for n in ("k", "kd") if inp[n] is not None)
    assert torch.allclose(lhs, rhs, atol=1e-10)
    # sum_d do*o == delta and sum over keys of ds == 0  =>  <q,dq> consistent with scale-derivative
    # (d loss / d scale) * scale == <q, dq>
    sc = torch.tensor(0.41, dtype=D64, requires_grad=True)
    o, _ = oracle.moda_dense(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], sc, G, mode, cb, dtype=D64)
    (o * inp["do"]).sum().backward()
    assert torch.allclose(sc.grad * 0.41, lhs, atol=1e-10)


@pytest.mark.parametrize("case", ORACLE_SMALL)
def test_blockwise_equals_dense(case):
    B, T, H, D, L, G, mode, cb = case
    inp = _inputs(B, T, H, D, L, G, mode, seed=29)
    a = oracle.moda_dense_fwd_bwd(inp, 0.29, G, mode, cb, dtype=D64)
    for block_rows in (G, 4 * G, 1024):
        b = oracle.moda_blockwise_fwd_bwd(inp, 0.29, G, mode, cb, block_rows=block_rows, dtype=D64)
        for n in ("o", "lse", "dq", "dk", "dv", "dkd", "dvd"):
            if a[n] is None:
                assert b[n] is None
            else:
                assert torch.allclose(a[n], b[n], atol=1e-11, rtol=1e-9), (n, block_rows)


def test_rows_subset_is_row_local():
    inp = _inputs(1, 12, 2, 8, 3, 2, "chunk_visible", seed=31)
    full = oracle.moda_dense_fwd_bwd(inp, 0.5, 2, "chunk_visible", 4, dtype=D64)
    rows = torch.tensor([0, 5, 6, 23])
    sub = oracle.moda_rows_subset(inp, rows, 0.5, 2, "chunk_visible", 4, dtype=D64)
    for n in ("o", "dq"):
        assert torch.allclose(sub[n], full[n][:, rows], atol=1e-12)
    assert torch.allclose(sub["lse"], full["lse"][:, rows], atol=1e-12)


def test_gradcheck_dense():
    inp = _inputs(1, 4, 1, 4, 2, 2, "causal", seed=37)
    args = [inp[n].clone().requires_grad_(True) for n in ("q", "k", "v", "kd", "vd")]
    fn = lambda q, k, v, kd, vd: oracle.moda_dense(q, k, v, kd, vd, 0.6, 2, "causal", dtype=D64)[0]
    assert torch.autograd.gradcheck(fn, args, eps=1e-6, atol=1e-6)


def test_depth_slot_permutation_invariance():
    """Permuting a token's L slots leaves o unchanged and permutes dkd/dvd rows."""
    B, T, H, D, L, G = 1, 6, 1, 8, 4, 2
    inp = _inputs(B, T, H, D, L, G, "causal", seed=41)
    perm = torch.tensor([2, 0, 3, 1])
    inp2 = dict(inp)
    inp2["kd"] = inp["kd"].view(B, T, L, H, D)[:, :, perm].reshape(B, T * L, H, D)
    inp2["vd"] = inp["vd"].view(B, T, L, H, D)[:, :, perm].reshape(B, T * L, H, D)
    a = oracle.moda_dense_fwd_bwd(inp, None, G, "causal", dtype=D64)
    b = oracle.moda_dense_fwd_bwd(inp2, None, G, "causal", dtype=D64)
    assert torch.allclose(a["o"], b["o"], atol=1e-12)
    assert torch.allclose(a["dkd"].view(B, T, L, H, D)[:, :, perm], b["dkd"].view(B, T, L, H, D), atol=1e-12)


def test_gqa_fold_equals_head_dim_gqa():
    """Folded [B,T*G,Hkv,D] with L=0 == plain attention over G*Hkv heads after the caller's reshape
    (vision_tasks/deit/models.py:248-250: group-major head order)."""
    B, T, Hkv, D, G = 1, 7, 2, 8, 3
    inp = _inputs(B, T, Hkv, D, 0, G, "causal", seed=43)
    o, _ = oracle.moda_dense(inp["q"], inp["k"], inp["v"], None, None, None, G, "causal", dtype=D64)
    q5 = inp["q"].view(B, T, G, Hkv, D)
    for g in range(G):
        ref = F.scaled_dot_product_attention(q5[:, :, g].permute(0, 2, 1, 3), inp["k"].permute(0, 2, 1, 3),
                                             inp["v"].permute(0, 2, 1, 3), is_causal=True)
        assert torch.allclose(o.view(B, T, G, Hkv, D)[:, :, g], ref.permute(0, 2, 1, 3), atol=1e-12)


def test_plain_gqa_matches_sdpa():
    gen = torch.Generator().manual_seed(47)
    q = torch.randn(2, 9, 6, 8, generator=gen, dtype=D64)
    k = torch.randn(2, 9, 2, 8, generator=gen, dtype=D64)
    v = torch.randn(2, 9, 2, 8, generator=gen, dtype=D64)
    o, _ = oracle.plain_gqa_dense(q, k, v, dtype=D64)
    ref = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3).repeat_interleave(3, 1),
                                         v.permute(0, 2, 1, 3).repeat_interleave(3, 1), is_causal=True)
    assert torch.allclose(o, ref.permute(0, 2, 1, 3), atol=1e-12)


def test_plain_gqa_lse_is_log2_of_the_row_sum():
    """The comparator's second output: 2**lse must be the row sum of 2**(scale*log2(e)*<q,k>) over the visible
    keys, computed here element by element without any library softmax."""
    gen = torch.Generator().manual_seed(53)
    B, T, Hq, Hkv, D = 2, 7, 6, 2, 8
    q = torch.randn(B, T, Hq, D, generator=gen, dtype=D64)
    k = torch.randn(B, T, Hkv, D, generator=gen, dtype=D64)
    v = torch.randn(B, T, Hkv, D, generator=gen, dtype=D64)
    _, lse = oracle.plain_gqa_dense(q, k, v, scale=0.37, dtype=D64)
    assert lse.shape == (B, T, Hq)
    for b in range(B):
        for h in range(Hq):
            for t in range(T):
                tot = sum(math.exp(0.37 * float(q[b, t, h] @ k[b, j, h // (Hq // Hkv)])) for j in range(t + 1))
                assert abs(2.0 ** float(lse[b, t, h]) - tot) <= 1e-9 * tot
    # and it is the folded operator's lse after the kv-major regrouping of heads (query head hq -> kv head hq // G)
    G = Hq // Hkv
    qf = q.view(B, T, Hkv, G, D).permute(0, 1, 3, 2, 4).reshape(B, T * G, Hkv, D)
    _, lse_f = oracle.moda_dense(qf, k, v, None, None, 0.37, G, "causal", dtype=D64)
    assert torch.allclose(lse_f.view(B, T, G, Hkv).permute(0, 1, 3, 2).reshape(B, T, Hq), lse, atol=1e-12)


@pytest.mark.parametrize("case", [(1, 24, 2, 8, 3, 2, "causal", 0), (1, 24, 1, 8, 2, 2, "chunk_visible", 4),
                                  (2, 10, 2, 8, 3, 1, "noncausal", 0), (1, 12, 2, 8, 4, 2, "depth_only", 0)])
def test_blockwise_token_range_and_rounded_o(case):
    """The two optional branches of the tiled form.  token_range=(a, b): the rows of those tokens equal the full
    evaluation's, and the key-side gradients equal those of a loss that only counts those rows (dO zeroed
    elsewhere).  o_round_dtype: delta is taken from o rounded to that type, i.e. the result equals the
    closed-form gradients with delta = sum(round(o) * do)."""
    B, T, H, D, L, G, mode, cb = case
    inp = _inputs(B, T, H, D, L, G, mode, seed=59)
    a, b = (8, 20) if T >= 24 else (4, 8)
    part = oracle.moda_blockwise_fwd_bwd(inp, 0.31, G, mode, cb, block_rows=4 * G, dtype=D64, token_range=(a, b))
    masked = dict(inp)
    masked["do"] = inp["do"].clone()
    masked["do"][:, :a * G] = 0
    masked["do"][:, b * G:] = 0
    full = oracle.moda_dense_fwd_bwd(masked, 0.31, G, mode, cb, dtype=D64)
    for n in ("o", "lse", "dq"):
        assert torch.allclose(part[n][:, a * G:b * G], full[n][:, a * G:b * G], atol=1e-11), n
    for n in ("dk", "dv", "dkd", "dvd"):
        if full[n] is not None:
            assert torch.allclose(part[n], full[n], atol=1e-11), n
    # rounded o: compare with the explicit formulas evaluated densely
    r = oracle.moda_blockwise_fwd_bwd(inp, 0.31, G, mode, cb, block_rows=4 * G, dtype=D64, o_round_dtype=torch.bfloat16)
    exact = oracle.moda_dense_fwd_bwd(inp, 0.31, G, mode, cb, dtype=D64)
    assert torch.allclose(r["o"], exact["o"], atol=1e-12)            # o itself is returned unrounded
    # d(delta) = sum((round(o) - o) * do) per row shifts ds by -p * d(delta): dq changes by -d(delta) * scale * sum_j p_j key_j
    ddelta = ((exact["o"].to(torch.bfloat16).to(D64) - exact["o"]) * inp["do"]).sum(-1)      # [B, rows, H]
    assert ddelta.abs().max() > 0
    q = inp["q"].clone().requires_grad_(True)
    _, lse = oracle.moda_dense(q, inp["k"], inp["v"], inp["kd"], inp["vd"], 0.31, G, mode, cb, dtype=D64)
    # sum_j p_j * scale * key_j = d(lse_natural)/dq, and lse is returned in base 2
    (lse * math.log(2.0) * (-ddelta)).sum().backward()
    assert torch.allclose(r["dq"], exact["dq"] + q.grad, atol=1e-10)


def test_depth_cache_layout():
    layers = [torch.full((2, 3, 2, 4), float(l)) + torch.arange(3).view(1, 3, 1, 1) * 10 for l in range(5)]
    c = oracle.depth_cache_ref(layers)
    assert c.shape == (2, 15, 2, 4)
    for t in range(3):
        for l in range(5):
            assert torch.all(c[:, t * 5 + l] == 10 * t + l)
    back = oracle.depth_cache_grad_ref(c, 5)
    for l in range(5):
        assert torch.equal(back[l], layers[l])


def test_flops_formula():
    # brute-force pair counts
    for (T, G, L, mode, cb) in [(9, 2, 3, "causal", 0), (9, 1, 2, "noncausal", 0), (10, 2, 3, "chunk_visible", 4),
                                (5, 4, 2, "depth_only", 0)]:
        pairs = int(oracle.visible_mask(T, G, L, mode, cb).sum()) // G
        assert oracle.flops_fwd(1, T, 1, 1, L, mode, cb) == 4 * pairs


def test_golden_fixture_matches_oracle():
    """The committed fixture (written by tests/golden/make_golden.py with the fp64 row loops) still matches."""
    import os

    import numpy as np

    path = os.path.join(os.path.dirname(__file__), "golden", "moda_small.npz")
    z = np.load(path)
    for mode, cb in (("causal", 0), ("noncausal", 0), ("chunk_visible", 4), ("depth_only", 0)):
        meta = z[f"{mode}_meta"]
        B, T, H, D, L, G, seed = (int(x) for x in meta)
        inp = oracle.make_inputs(B, T, H, D, L, G, seed=seed, dtype=torch.float32, std=0.5,
                                 depth_only=(mode == "depth_only"))
        r = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, mode, cb, dtype=torch.float64)
        for n in ("o", "lse", "dq", "dk", "dv", "dkd", "dvd"):
            key = f"{mode}_{n}"
            if r[n] is None:
                assert key not in z
            else:
                assert np.allclose(z[key], r[n].numpy(), atol=1e-6), key


def test_compact_and_scatter_depth_are_adjoint_slot_selections():
    """compact_depth keeps exactly rows t*L + l with l < valid, in order; scatter_depth_grad is its
    transpose (checked against autograd and against a literal index loop)."""
    B, T, L, H, D, valid = 2, 5, 4, 3, 2, 3
    x = torch.arange(B * T * L * H * D, dtype=torch.float64).reshape(B, T * L, H, D).requires_grad_(True)
    c = oracle.compact_depth(x, T, valid)
    assert c.shape == (B, T * valid, H, D)
    for t in range(T):
        for l in range(valid):
            assert torch.equal(c[:, t * valid + l], x[:, t * L + l])
    w = torch.randn_like(c)
    (c * w).sum().backward()
    assert torch.equal(x.grad, oracle.scatter_depth_grad(w, T, L))
    for t in range(T):
        for l in range(valid, L):
            assert x.grad[:, t * L + l].abs().max() == 0


@pytest.mark.parametrize("mode,G,L,cb", [("causal", 1, 2, 0), ("causal", 2, 3, 0), ("noncausal", 2, 1, 0),
                                          ("chunk_visible", 2, 2, 2), ("depth_only", 2, 3, 0), ("causal", 1, 0, 0)])
def test_packed_batch_is_block_masked_attention_over_the_packed_axis(mode, G, L, cb):
    """The per-sequence evaluation that defines cu_seqlens equals ONE library softmax over the whole packed
    axis under a mask written out element by element (same sequence AND the variant's rule on positions
    counted from the sequence start), forward and all gradients: pins which rows belong to which
    sequence (q rows cu*G, depth rows cu*L)."""
    cu = [0, 3, 3, 4, 9]  # lengths 3, 0, 1, 5
    total, H, D = cu[-1], 2, 8
    g = torch.Generator().manual_seed(11)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    inp = {"q": r(1, total * G, H, D), "do": r(1, total * G, H, D)}
    if mode != "depth_only":
        inp["k"], inp["v"] = r(1, total, H, D), r(1, total, H, D)
    if L:
        inp["kd"], inp["vd"] = r(1, total * L, H, D), r(1, total * L, H, D)
    scale = 0.3
    got = oracle.moda_packed_fwd_bwd(inp, cu, scale, G, mode, cb, dtype=torch.float64)

    mask = oracle.packed_visible_mask(cu, G, L, mode, cb)
    leaf = {n: x.clone().requires_grad_(True) for n, x in inp.items() if n != "do"}
    keys = [leaf["k"] if "k" in leaf else torch.zeros(1, total, H, D, dtype=torch.float64)]
    vals = [leaf["v"] if "v" in leaf else torch.zeros(1, total, H, D, dtype=torch.float64)]
    if L:
        keys.append(leaf["kd"])
        vals.append(leaf["vd"])
    kc, vc = torch.cat(keys, 1).transpose(1, 2), torch.cat(vals, 1).transpose(1, 2)
    o = F.scaled_dot_product_attention(leaf["q"].transpose(1, 2), kc, vc, attn_mask=mask.view(1, 1, *mask.shape),
                                       scale=scale).transpose(1, 2)
    (o * inp["do"]).sum().backward()
    assert torch.allclose(got["o"], o.detach(), atol=1e-12)
    for n in ("q", "k", "v", "kd", "vd"):
        if n in leaf:
            assert torch.allclose(got["d" + n], leaf[n].grad, atol=1e-11), n
    logits = torch.einsum("bqhd,bhkd->bhqk", inp["q"], kc.detach()) * scale
    lse = torch.logsumexp(logits.masked_fill(~mask, float("-inf")), -1).permute(0, 2, 1) / math.log(2.0)
    assert torch.allclose(got["lse"], lse, atol=1e-12)
