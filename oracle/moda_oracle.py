"""Oracle for the fused sequence+depth attention path (test infrastructure).

This file restates, in plain torch on the CPU, the algorithm that the
reference defines with its naive torch loops.  It is the checker for the HIP
kernels and is never on the product path.

Reference text followed (read, never imported):
  * MoDA causal / non-causal:  libs/moda_triton/fla/ops/moda/moda_v14.py:1845-1846
    (``_ref_seq_kv_limit``) and :1900-1991 (``naive_mixture_of_depth_causal_ref``)
  * chunk-visible MoDA:        libs/moda_triton/fla/ops/moda/moda_v16.py:2487-2582
  * depth-only (FDA):          libs/moda_triton/fla/ops/moda/fda_v12.py:1143-1196
  * test-side pass rule:       libs/moda_triton/tests/ops/test_moda.py:84-92
  * depth cache layout:        vision_tasks/deit/models.py:361-375
  * plain GQA comparator:      libs/moda_triton/fla/ops/attn/parallel.py:678-730

Three forms of the same function are kept so that each pins the others:
  (i)   ``moda_rows``      literal per-row loops (the reference's own shape),
  (ii)  ``moda_dense``     one masked softmax over the concatenated
                           ``[sequence | depth]`` key axis (autograd gives grads),
  (iii) ``moda_blockwise_fwd_bwd``  tiled fp32 evaluation with explicit
                           gradient formulas for long sequences.
Pinning (tests/test_oracle.py): (ii) against
``torch.nn.functional.scaled_dot_product_attention`` with the same boolean
mask, (i) against (ii), (iii) against (ii), special cases with textbook closed
forms (L=0 -> causal SDPA, replicated depth slots -> +log(1+L) on the diagonal
logit, constant V -> constant O), sum invariants of the gradients and
``torch.autograd.gradcheck`` in fp64.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence, Tuple

import torch

MODES = ("causal", "noncausal", "chunk_visible", "depth_only")
LN2 = math.log(2.0)


# --------------------------------------------------------------------------
# visible set
# --------------------------------------------------------------------------
def visible_mask(
    T: int,
    G: int,
    L: int,
    mode: str,
    chunk_tokens: int = 0,
    rows: Optional[torch.Tensor] = None,
    device=None,
) -> torch.Tensor:
    """Boolean mask ``[rows, T + T*L]`` over the concatenated key axis.

    Row ``r`` belongs to base token ``t = r // G``.  Sequence column ``j`` is
    visible iff ``j <= t`` (causal, chunk_visible; moda_v14.py:1845-1846), always
    (noncausal), never (depth_only, fda_v12.py:1143-1196).  Depth column ``c``
    (owner token ``c // L``) is visible iff ``c // L == t`` (moda_v14.py:1965) or,
    chunk-visible, ``floor(t / Cb) * Cb <= c // L <= t`` (moda_v16.py:2557-2561).
    """
    assert mode in MODES
    if rows is None:
        rows = torch.arange(T * G, device=device)
    t = (rows // G).view(-1, 1)
    j = torch.arange(T, device=rows.device).view(1, -1)
    if mode in ("causal", "chunk_visible"):
        seq = j <= t
    elif mode == "noncausal":
        seq = torch.ones(rows.numel(), T, dtype=torch.bool, device=rows.device)
    else:
        seq = torch.zeros(rows.numel(), T, dtype=torch.bool, device=rows.device)
    if L == 0:
        return seq
    owner = (torch.arange(T * L, device=rows.device) // L).view(1, -1)
    if mode == "chunk_visible":
        assert chunk_tokens >= 1
        start = (t // chunk_tokens) * chunk_tokens
        dep = (owner >= start) & (owner <= t)
    else:
        dep = owner == t
    return torch.cat([seq, dep], dim=1)


# --------------------------------------------------------------------------
# (i) literal per-row loops
# --------------------------------------------------------------------------
def moda_rows(
    q: torch.Tensor,
    k: Optional[torch.Tensor],
    v: Optional[torch.Tensor],
    kd: Optional[torch.Tensor] = None,
    vd: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    moda_group_num: int = 1,
    mode: str = "causal",
    chunk_tokens: int = 0,
    dtype=torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-(b, h, row) loops in the order the reference writes them.

    Returns ``(out, lse)`` with ``lse`` in base-2 units
    (``logsumexp(logits) / ln 2``, moda_v14.py:1989).
    """
    assert mode in MODES
    B, Tq, H, D = q.shape
    G = moda_group_num
    assert Tq % G == 0
    T = Tq // G
    use_depth = kd is not None and vd is not None
    if mode == "depth_only":
        assert use_depth
    L = kd.shape[1] // T if use_depth else 0
    Dv = (vd if use_depth else v).shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = torch.empty(B, Tq, H, Dv, dtype=dtype)
    lse = torch.empty(B, Tq, H, dtype=dtype)
    for b in range(B):
        for h in range(H):
            q_bh = q[b, :, h].to(dtype)
            if mode != "depth_only":
                k_bh = k[b, :, h].to(dtype)
                v_bh = v[b, :, h].to(dtype)
            if use_depth:
                kd_bh = kd[b, :, h].to(dtype).view(T, L, D)
                vd_bh = vd[b, :, h].to(dtype).view(T, L, Dv)
            for r in range(Tq):
                t = r // G
                qv = q_bh[r]
                parts_l, parts_v = [], []
                if mode != "depth_only":
                    end = t + 1 if mode in ("causal", "chunk_visible") else T
                    parts_l.append((qv @ k_bh[:end].T) * scale)
                    parts_v.append(v_bh[:end])
                if use_depth:
                    if mode == "chunk_visible":
                        s0 = (t // chunk_tokens) * chunk_tokens
                        ksel = kd_bh[s0 : t + 1].reshape(-1, D)
                        vsel = vd_bh[s0 : t + 1].reshape(-1, Dv)
                    else:
                        ksel, vsel = kd_bh[t], vd_bh[t]
                    parts_l.append((ksel @ qv) * scale)
                    parts_v.append(vsel)
                logits = torch.cat(parts_l, dim=0)
                vals = torch.cat(parts_v, dim=0)
                w = torch.softmax(logits, dim=0)
                out[b, r, h] = (w.unsqueeze(1) * vals).sum(0)
                lse[b, r, h] = torch.logsumexp(logits, dim=0) / LN2
    return out, lse


# --------------------------------------------------------------------------
# (ii) dense masked softmax over [seq | depth]
# --------------------------------------------------------------------------
def moda_dense(
    q: torch.Tensor,
    k: Optional[torch.Tensor],
    v: Optional[torch.Tensor],
    kd: Optional[torch.Tensor] = None,
    vd: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    moda_group_num: int = 1,
    mode: str = "causal",
    chunk_tokens: int = 0,
    dtype=torch.float32,
    rows: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same function as :func:`moda_rows`, vectorised and differentiable.

    ``rows`` optionally restricts evaluation to a subset of folded query rows
    (each row's output depends only on that row of ``q``), in which case ``q``
    must already hold just those rows.
    """
    assert mode in MODES
    B, Tq_in, H, D = q.shape
    G = moda_group_num
    use_depth = kd is not None and vd is not None
    if mode == "depth_only":
        assert use_depth
        if rows is not None:
            raise ValueError("rows= is not supported for depth_only (T is inferred from the full q)")
        T = Tq_in // G
    else:
        T = k.shape[1]
    L = kd.shape[1] // T if use_depth else 0
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    keys, vals = [], []
    if mode != "depth_only":
        keys.append(k.to(dtype))
        vals.append(v.to(dtype))
    else:
        # keep the mask width T + T*L: prepend T dummy columns that are never visible
        keys.append(torch.zeros(B, T, H, D, dtype=dtype, device=q.device))
        vals.append(torch.zeros(B, T, H, vd.shape[-1], dtype=dtype, device=q.device))
    if use_depth:
        keys.append(kd.to(dtype))
        vals.append(vd.to(dtype))
    kc = torch.cat(keys, dim=1)
    vc = torch.cat(vals, dim=1)
    mask = visible_mask(T, G, L, mode, chunk_tokens, rows=rows, device=q.device)
    logits = torch.einsum("bqhd,bkhd->bhqk", q.to(dtype), kc) * scale
    logits = logits.masked_fill(~mask.view(1, 1, *mask.shape), float("-inf"))
    lse = torch.logsumexp(logits, dim=-1)
    p = torch.exp(logits - lse.unsqueeze(-1))
    out = torch.einsum("bhqk,bkhd->bqhd", p, vc)
    return out, (lse / LN2).permute(0, 2, 1)


def moda_dense_fwd_bwd(inp: Dict[str, torch.Tensor], scale, G, mode, chunk_tokens=0, dtype=torch.float32):
    """Forward + autograd backward of form (ii).

    ``inp`` holds q, k, v, kd, vd, do (any may be None except q/do).  The loss
    is ``sum(out * do)`` as in test_moda.py:271-272.  Returns a dict with
    o, lse, dq, dk, dv, dkd, dvd (None where the input was None).
    """
    leaf = {}
    for name in ("q", "k", "v", "kd", "vd"):
        x = inp.get(name)
        leaf[name] = None if x is None else x.detach().to(dtype).clone().requires_grad_(True)
    o, lse = moda_dense(leaf["q"], leaf["k"], leaf["v"], leaf["kd"], leaf["vd"], scale, G, mode, chunk_tokens, dtype)
    (o * inp["do"].to(dtype)).sum().backward()
    res = {"o": o.detach(), "lse": lse.detach()}
    for name in ("q", "k", "v", "kd", "vd"):
        res["d" + name] = None if leaf[name] is None else leaf[name].grad
    return res


def moda_rows_subset(inp, rows: torch.Tensor, scale, G, mode, chunk_tokens=0, dtype=torch.float32):
    """o, lse and dq for a subset of folded query rows (row-local quantities)."""
    qs = inp["q"][:, rows].detach().to(dtype).clone().requires_grad_(True)
    o, lse = moda_dense(qs, inp.get("k"), inp.get("v"), inp.get("kd"), inp.get("vd"), scale, G, mode,
                        chunk_tokens, dtype, rows=rows)
    (o * inp["do"][:, rows].to(dtype)).sum().backward()
    return {"o": o.detach(), "lse": lse.detach(), "dq": qs.grad}


# --------------------------------------------------------------------------
# partially filled depth stream (an extension of this build; no reference counterpart)
# --------------------------------------------------------------------------
def compact_depth(x: torch.Tensor, T: int, valid: int) -> torch.Tensor:
    """``[B, T*L, H, D]`` -> ``[B, T*valid, H, D]`` keeping slots ``l < valid`` of every token.

    This DEFINES the ``depth_valid`` option of the kernels: with ``depth_valid = valid`` they must
    return what the functions of this file return for the compacted tensors (the layout is that of
    vision_tasks/deit/models.py:361-375: row ``t*L + l`` = slot ``l`` of token ``t``)."""
    B, TL, H, D = x.shape
    L = TL // T
    return x.reshape(B, T, L, H, D)[:, :, :valid].reshape(B, T * valid, H, D)


def scatter_depth_grad(g: torch.Tensor, T: int, L: int) -> torch.Tensor:
    """Gradient w.r.t. the compacted depth tensor -> gradient w.r.t. the ``L``-slot tensor (zeros in
    the slots that were dropped)."""
    B, TV, H, D = g.shape
    valid = TV // T
    out = torch.zeros(B, T, L, H, D, dtype=g.dtype, device=g.device)
    out[:, :, :valid] = g.reshape(B, T, valid, H, D)
    return out.reshape(B, T * L, H, D)


# --------------------------------------------------------------------------
# packed variable-length batches (an extension of this build; the reference carries a cu_seqlens
# argument but asserts it away, moda_v14.py:2672-2673)
# --------------------------------------------------------------------------
def packed_visible_mask(cu: Sequence[int], G: int, L: int, mode: str, chunk_tokens: int = 0) -> torch.Tensor:
    """Boolean mask ``[total*G, total + total*L]`` of a packed batch, written out element by element.

    ``cu`` are cumulative sequence lengths in base tokens.  A query row sees a column iff both belong to
    the same sequence and the rule of :func:`visible_mask` holds for their positions counted from the
    sequence's first token (so chunks of the chunk-visible variant restart with every sequence)."""
    total = int(cu[-1])
    seq_of, local = [], []
    for i in range(len(cu) - 1):
        for t in range(int(cu[i]), int(cu[i + 1])):
            seq_of.append(i)
            local.append(t - int(cu[i]))
    m = torch.zeros(total * G, total + total * L, dtype=torch.bool)
    for r in range(total * G):
        t = r // G
        for j in range(total):
            if seq_of[j] != seq_of[t]:
                continue
            if mode in ("causal", "chunk_visible"):
                m[r, j] = local[j] <= local[t]
            elif mode == "noncausal":
                m[r, j] = True
        for c in range(total * L):
            w = c // L
            if seq_of[w] != seq_of[t]:
                continue
            if mode == "chunk_visible":
                start = (local[t] // chunk_tokens) * chunk_tokens
                m[r, total + c] = start <= local[w] <= local[t]
            else:
                m[r, total + c] = w == t
    return m


def moda_packed_fwd_bwd(inp: Dict[str, torch.Tensor], cu: Sequence[int], scale, G, mode, chunk_tokens=0,
                        dtype=torch.float32):
    """:func:`moda_dense_fwd_bwd` for a packed batch: tensors of batch size 1 hold the sequences back to
    back (sequence i = base tokens ``cu[i] .. cu[i+1]``, query rows ``cu*G``, depth rows ``cu*L``); every
    sequence is evaluated on its own and the results are put back in place.  This DEFINES the
    ``cu_seqlens`` option of the kernels."""
    total = int(cu[-1])
    L = inp["kd"].shape[1] // total if (inp.get("kd") is not None and total > 0) else 0
    span = {"q": G, "do": G, "k": 1, "v": 1, "kd": L, "vd": L}
    res = {}
    for name in ("o", "dq"):
        res[name] = torch.zeros(inp["q"].shape, dtype=dtype)
    res["lse"] = torch.zeros(inp["q"].shape[:3], dtype=dtype)
    for name in ("k", "v", "kd", "vd"):
        res["d" + name] = None if inp.get(name) is None else torch.zeros(inp[name].shape, dtype=dtype)
    for i in range(len(cu) - 1):
        a, b = int(cu[i]), int(cu[i + 1])
        if a == b:
            continue
        part = {n: (None if inp.get(n) is None else inp[n][:, a * m:b * m]) for n, m in span.items()}
        r = moda_dense_fwd_bwd(part, scale, G, mode, chunk_tokens, dtype)
        res["o"][:, a * G:b * G] = r["o"]
        res["lse"][:, a * G:b * G] = r["lse"]
        res["dq"][:, a * G:b * G] = r["dq"]
        for n in ("k", "v", "kd", "vd"):
            if r["d" + n] is not None:
                res["d" + n][:, a * span[n]:b * span[n]] = r["d" + n]
    return res


# --------------------------------------------------------------------------
# (iii) blockwise evaluation with explicit gradient formulas
# --------------------------------------------------------------------------
@torch.no_grad()
def moda_blockwise_fwd_bwd(inp, scale, G, mode, chunk_tokens=0, block_rows=4096, dtype=torch.float32,
                           o_round_dtype=None, token_range=None):
    """Tiled evaluation for long sequences; runs on whatever device ``inp`` is on.

    Uses the closed-form gradients of softmax attention
    (``ds = p * (dp - delta)``, ``delta = sum(o * do)``) instead of autograd so
    that only ``block_rows x keys`` scores are alive at a time.  ``o_round_dtype``
    optionally rounds ``o`` before ``delta`` as the kernels do (moda_v14.py:525-539
    reads the stored, rounded ``o``).  ``token_range=(a, b)`` evaluates only the query rows of tokens
    ``a <= t < b`` (outputs of other rows are left unset, key gradients hold only those rows'
    contributions); used to time a bounded sample of a large workload.
    """
    q, k, v, kd, vd, do = (inp.get(n) for n in ("q", "k", "v", "kd", "vd", "do"))
    B, Tq, H, D = q.shape
    T = Tq // G
    use_depth = kd is not None
    L = kd.shape[1] // T if use_depth else 0
    dev = q.device
    f = lambda x: None if x is None else x.to(dtype)
    q, k, v, kd, vd, do = map(f, (q, k, v, kd, vd, do))
    Dv = (vd if use_depth else v).shape[-1]
    o = torch.empty(B, Tq, H, Dv, dtype=dtype, device=dev)
    lse = torch.empty(B, Tq, H, dtype=dtype, device=dev)
    dq = torch.zeros_like(q)
    dk = None if k is None else torch.zeros_like(k)
    dv = None if v is None else torch.zeros_like(v)
    dkd = None if kd is None else torch.zeros_like(kd)
    dvd = None if vd is None else torch.zeros_like(vd)
    if use_depth:
        kd5 = kd.view(B, T, L, H, D)
        vd5 = vd.view(B, T, L, H, Dv)
        dkd5 = dkd.view(B, T, L, H, D)
        dvd5 = dvd.view(B, T, L, H, Dv)
    step_tok = max(1, block_rows // G)
    if mode == "chunk_visible":
        step_tok = max(chunk_tokens, (step_tok // chunk_tokens) * chunk_tokens)
    tok_a, tok_b = (0, T) if token_range is None else token_range
    if mode == "chunk_visible":
        assert tok_a % chunk_tokens == 0
    for t0 in range(tok_a, tok_b, step_tok):
        t1 = min(tok_b, t0 + step_tok)
        r0, r1 = t0 * G, t1 * G
        rows = torch.arange(r0, r1, device=dev)
        tok = rows // G
        qb = q[:, r0:r1]
        logit_parts, val_parts = [], []
        send = 0
        if mode != "depth_only":
            send = t1 if mode in ("causal", "chunk_visible") else T
            ls = torch.einsum("bqhd,bkhd->bhqk", qb, k[:, :send]) * scale
            if mode in ("causal", "chunk_visible"):
                m = torch.arange(send, device=dev).view(1, -1) <= tok.view(-1, 1)
                ls = ls.masked_fill(~m.view(1, 1, *m.shape), float("-inf"))
            logit_parts.append(ls)
        if use_depth:
            # depth keys of tokens [d0, t1) flattened; d0 = chunk start of t0 for chunk-visible
            d0 = (t0 // chunk_tokens) * chunk_tokens if mode == "chunk_visible" else t0
            kdb = kd5[:, d0:t1].reshape(B, (t1 - d0) * L, H, D)
            vdb = vd5[:, d0:t1].reshape(B, (t1 - d0) * L, H, Dv)
            ld = torch.einsum("bqhd,bkhd->bhqk", qb, kdb) * scale
            owner = d0 + torch.arange((t1 - d0) * L, device=dev) // L
            if mode == "chunk_visible":
                st = (tok // chunk_tokens) * chunk_tokens
                m = (owner.view(1, -1) >= st.view(-1, 1)) & (owner.view(1, -1) <= tok.view(-1, 1))
            else:
                m = owner.view(1, -1) == tok.view(-1, 1)
            ld = ld.masked_fill(~m.view(1, 1, *m.shape), float("-inf"))
            logit_parts.append(ld)
        logits = torch.cat(logit_parts, dim=-1)
        lse_b = torch.logsumexp(logits, dim=-1)
        p = torch.exp(logits - lse_b.unsqueeze(-1))
        ps, pd = p[..., :send], p[..., send:]
        ob = torch.zeros(B, r1 - r0, H, Dv, dtype=dtype, device=dev)
        if send:
            ob += torch.einsum("bhqk,bkhd->bqhd", ps, v[:, :send])
        if use_depth:
            ob += torch.einsum("bhqk,bkhd->bqhd", pd, vdb)
        o[:, r0:r1] = ob
        lse[:, r0:r1] = (lse_b / LN2).permute(0, 2, 1)
        dob = do[:, r0:r1]
        o_for_delta = ob if o_round_dtype is None else ob.to(o_round_dtype).to(dtype)
        delta = (o_for_delta * dob).sum(-1).permute(0, 2, 1)  # b h q
        if send:
            dps = torch.einsum("bqhd,bkhd->bhqk", dob, v[:, :send])
            dss = ps * (dps - delta.unsqueeze(-1))
            dq[:, r0:r1] += torch.einsum("bhqk,bkhd->bqhd", dss, k[:, :send]) * scale
            dk[:, :send] += torch.einsum("bhqk,bqhd->bkhd", dss, qb) * scale
            dv[:, :send] += torch.einsum("bhqk,bqhd->bkhd", ps, dob)
        if use_depth:
            dpd = torch.einsum("bqhd,bkhd->bhqk", dob, vdb)
            dsd = pd * (dpd - delta.unsqueeze(-1))
            dq[:, r0:r1] += torch.einsum("bhqk,bkhd->bqhd", dsd, kdb) * scale
            dkd5[:, d0:t1] += (torch.einsum("bhqk,bqhd->bkhd", dsd, qb) * scale).view(B, t1 - d0, L, H, D)
            dvd5[:, d0:t1] += torch.einsum("bhqk,bqhd->bkhd", pd, dob).view(B, t1 - d0, L, H, Dv)
    return {"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}


# --------------------------------------------------------------------------
# plain GQA attention comparator (head-dim GQA, kv head = hq // G)
# --------------------------------------------------------------------------
def plain_gqa_dense(q, k, v, scale=None, causal=True, dtype=torch.float32):
    """Causal softmax attention with head-dim GQA as in fla/ops/attn/parallel.py:48-49
    (query head ``hq`` reads kv head ``hq // G``).  Returns (o, lse base-2)."""
    B, T, Hq, D = q.shape
    Hkv = k.shape[2]
    G = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    kk = k.to(dtype).repeat_interleave(G, dim=2)
    vv = v.to(dtype).repeat_interleave(G, dim=2)
    logits = torch.einsum("bqhd,bkhd->bhqk", q.to(dtype), kk) * scale
    if causal:
        m = torch.ones(T, T, dtype=torch.bool, device=q.device).tril()
        logits = logits.masked_fill(~m, float("-inf"))
    lse = torch.logsumexp(logits, dim=-1)
    p = torch.exp(logits - lse.unsqueeze(-1))
    return torch.einsum("bhqk,bkhd->bqhd", p, vv), (lse / LN2).permute(0, 2, 1)


# --------------------------------------------------------------------------
# depth cache layout (the "reorganisation")
# --------------------------------------------------------------------------
def depth_cache_ref(layers: Sequence[torch.Tensor]) -> torch.Tensor:
    """``[B,T,H,D]`` x L  ->  ``[B, T*L, H, D]`` with row ``t*L + l`` = layer l of token t
    (vision_tasks/deit/models.py:370-374)."""
    x = torch.stack(list(layers), dim=2)
    B, T, L, H, D = x.shape
    return x.reshape(B, T * L, H, D).contiguous()


def depth_cache_grad_ref(dcache: torch.Tensor, L: int):
    """Transpose of :func:`depth_cache_ref`: split ``[B,T*L,H,D]`` into L per-layer grads."""
    B, TL, H, D = dcache.shape
    x = dcache.view(B, TL // L, L, H, D)
    return [x[:, :, l].contiguous() for l in range(L)]


# --------------------------------------------------------------------------
# seeded inputs, metrics, algorithmic work
# --------------------------------------------------------------------------
def make_inputs(B, T, H, D, L, G=1, seed=0, dtype=torch.float32, std=1.0, do_std=1.0,
                prescale_q=False, depth_only=False, Hq=None, Dv=None):
    """Deterministic inputs from a CPU generator, drawn in fp32 in the order
    q, k, v, kd, vd, do and then cast.  ``Hq`` (plain GQA layout) makes q
    ``[B,T,Hq,D]`` instead of the folded ``[B,T*G,H,D]``; ``Dv`` gives v, vd and do a
    head dim of their own."""
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    qshape = (B, T, Hq, D) if Hq is not None else (B, T * G, H, D)
    Dv = D if Dv is None else Dv
    q = rn(*qshape) * std
    if prescale_q:
        q = q * (D ** -0.5)
    k = rn(B, T, H, D) * std
    v = rn(B, T, H, Dv) * std
    kd = rn(B, T * L, H, D) * std if L > 0 else None
    vd = rn(B, T * L, H, Dv) * std if L > 0 else None
    do = rn(*qshape[:3], Dv) * do_std
    c = lambda x: None if x is None else x.to(dtype)
    out = {"q": c(q), "k": c(k), "v": c(v), "kd": c(kd), "vd": c(vd), "do": c(do)}
    if depth_only:
        out["k"] = out["v"] = None
    return out


def error_metrics(x, ref):
    """(max_abs, l2_rel) as in test_moda.py:84-92."""
    diff = (x.double() - ref.double())
    max_abs = diff.abs().max().item() if diff.numel() else 0.0
    l2_rel = (diff.pow(2).sum().sqrt() / (ref.double().pow(2).sum().sqrt() + 1e-12)).item()
    return max_abs, l2_rel


def passes_reference_rule(x, ref, atol=1e-2, rtol=1e-2):
    """``max_abs <= atol or l2_rel <= 10*rtol`` (test_moda.py:84-92, 298-299)."""
    max_abs, l2_rel = error_metrics(x, ref)
    return (max_abs <= atol) or (l2_rel <= 10 * rtol)


def flops_fwd(B, T, Hq, D, L, mode, chunk_tokens=0):
    """Algorithmic forward FLOPs: 4*D per visible (query, key) pair; masked tile work is not counted."""
    if mode in ("causal", "chunk_visible"):
        pseq = T * (T + 1) // 2
    elif mode == "noncausal":
        pseq = T * T
    else:
        pseq = 0
    if L == 0:
        pdep = 0
    elif mode == "chunk_visible":
        full, rem = divmod(T, chunk_tokens)
        pdep = L * (full * chunk_tokens * (chunk_tokens + 1) // 2 + rem * (rem + 1) // 2)
    else:
        pdep = T * L
    return 4 * D * B * Hq * (pseq + pdep)
