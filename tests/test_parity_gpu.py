"""GPU parity tests: HIP kernels (through the Python host, i.e. through the C ABI of
libmoda_hip.so) against the oracle on identical seeded inputs.

Tolerances (elementwise ``|got - ref| <= atol + rtol * |ref|``; the rtol term is one to
two units in the last place of the 16-bit output format and only matters for
gradient entries much larger than one):
    bf16 tensors : atol 2e-2, rtol 2**-7      fp16 tensors : atol 4e-3, rtol 2**-9
    fp32 tensors : atol 2e-4, rtol 1e-4       LSE (fp32, base 2): atol 1e-3
plus the reference's own rule ``max_abs <= 1e-2 or l2_rel <= 0.1``
(libs/moda_triton/tests/ops/test_moda.py:84-92) on its 102-case matrix.
"""
import math
import sys

import pytest
import torch

import oracle
from cases import REFERENCE_MATRIX

pytestmark = pytest.mark.gpu

TOL = {
    torch.bfloat16: (2e-2, 2.0 ** -7),
    torch.float16: (4e-3, 2.0 ** -9),
    torch.float32: (2e-4, 1e-4),
}
LSE_ATOL = 1e-3
MODE_ID = {"causal": 0, "noncausal": 1, "chunk_visible": 2, "depth_only": 3}


def say(msg):
    sys.stdout.write(msg + "\n")
    sys.stdout.flush()


def to_dev(inp, dev):
    return {k: (None if v is None else v.to(dev)) for k, v in inp.items()}


def check(name, got, ref, dtype, what=""):
    atol, rtol = TOL[dtype] if name != "lse" else (LSE_ATOL, 0.0)
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, (what, name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{what} {name}: non-finite values"
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    bad = err > bound
    if bad.any():
        i = torch.argmax(err - bound)
        raise AssertionError(
            f"{what} {name}: {int(bad.sum())} elements out of tolerance; worst |err|={err.flatten()[i]:.4e} "
            f"at ref={ref.flatten()[i]:.4e} (atol={atol}, rtol={rtol}); max_abs={err.max():.4e}")


def run_hip(inp, scale, G, mode, cb=0, row_sums_only=False, no_row_split=False):
    """``row_sums_only``: give the backward a workspace that holds the row sums and nothing else, which keeps the
    sequence dK/dV on the single-pass summation order (no row segments) and the depth gradients on the kernel that
    recomputes its scores.  ``no_row_split``: a workspace with room for the row sums and the depth scores the dQ kernel
    hands to the depth-gradient kernel, but not for partial sums (what a packed batch is given)."""
    from moda_amd import ops

    m = MODE_ID[mode]
    o, lse = ops._raw_fwd(m, inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], scale, G, cb)
    rows = inp["q"].shape[0] * inp["q"].shape[1] * inp["q"].shape[2]
    ws = None
    if row_sums_only:
        ws = torch.empty(max(4, 4 * rows), dtype=torch.uint8, device=inp["q"].device)
    elif no_row_split:
        up = lambda n: (n + 255) // 256 * 256
        slots = 0 if inp["kd"] is None else inp["kd"].shape[1] // (inp["q"].shape[1] // G)
        ws = torch.empty(up(4 * rows) + 2 * up(2 * rows * slots), dtype=torch.uint8, device=inp["q"].device)
    dq, dk, dv, dkd, dvd = ops._raw_bwd(m, inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], o, lse, inp["do"],
                                        scale, G, cb, ws=ws)
    return {"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}


L2_REL = {torch.bfloat16: 1e-2, torch.float16: 5e-3, torch.float32: 1e-4}


def check_l2(name, got, ref, dtype, what="", blocks=16):
    """Relative L2 error of the whole tensor and of each of `blocks` contiguous blocks of rows (dim 1): the
    elementwise rule's absolute term is larger than the late rows of a long causal sequence, whose outputs
    average over thousands of values; a per-block relative norm still sees an error confined to them."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    tol = L2_REL[dtype]
    n_rows = ref.shape[1]
    edges = sorted({(n_rows * i) // blocks for i in range(blocks + 1)})
    spans = [(0, n_rows)] + [(a, b) for a, b in zip(edges[:-1], edges[1:]) if b > a]
    for a, b in spans:
        r = ref[:, a:b]
        den = r.norm().item()
        num = (got[:, a:b] - r).norm().item()
        # a block whose true value is numerically zero has no relative error to speak of
        assert num <= tol * den or num <= 1e-3 * math.sqrt(max(r.numel(), 1)) * TOL[dtype][0], \
            f"{what} {name}: rows [{a},{b}) relative L2 error {num / max(den, 1e-30):.3e} > {tol}"


def numerics(got, ref):
    """max |err|, max |ref| and the relative L2 error of one tensor."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    return (got - ref).abs().max().item(), ref.abs().max().item(), ((got - ref).norm() / ref.norm().clamp_min(1e-30)).item()


def compare_all(got, ref, dtype, what, plain_atol=None):
    """``plain_atol``: additionally hold every tensor but lse to max |err| <= plain_atol with no relative term (the
    bar the benchmark configurations are quoted on) and print what was observed."""
    for n in ("o", "lse", "dq", "dk", "dv", "dkd", "dvd"):
        if ref[n] is None:
            assert got[n] is None, (what, n)
            continue
        check(n, got[n], ref[n], dtype, what)
        if n != "lse":
            check_l2(n, got[n], ref[n], dtype, what)
        if plain_atol is not None:
            err, mag, rel = numerics(got[n], ref[n])
            say(f"NUMERICS {what} {n}: max_abs_err={err:.3e} max_abs_ref={mag:.3e} rel_l2={rel:.3e}")
            assert err <= (LSE_ATOL if n == "lse" else plain_atol), f"{what} {n}: max |err| {err:.3e} > {plain_atol}"


# ---------------------------------------------------------------------------
# the reference's own 102-case matrix (causal, D=64), plus LSE which it never checked
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("idx", range(len(REFERENCE_MATRIX)))
def test_reference_matrix(gpu_device, idx):
    B, T, H, L, G, dt, scale = REFERENCE_MATRIX[idx]
    dtype = torch.float16 if dt == "h" else torch.bfloat16
    D = 64
    sc = scale if scale is not None else D ** -0.5
    say(f"[matrix {idx}] B{B} T{T} H{H} L{L} G{G} {dtype} scale={sc}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=2025 + idx, dtype=dtype)
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, "causal")
    got = run_hip(to_dev(inp, gpu_device), sc, G, "causal")
    for n in ("o", "dq", "dk", "dv", "dkd", "dvd"):
        if ref[n] is None:
            continue
        assert oracle.passes_reference_rule(got[n].float().cpu(), ref[n]), (idx, n)
        # tighter than the reference's rule; the absolute alternative covers tensors whose true value is
        # (numerically) zero, e.g. dk of a one-token sequence, where a relative error means nothing
        max_abs, l2 = oracle.error_metrics(got[n].float().cpu(), ref[n])
        assert l2 <= 1e-2 or max_abs <= 1e-3, (idx, n, l2, max_abs)
    check("lse", got["lse"], ref["lse"], dtype, f"matrix {idx}")


# ---------------------------------------------------------------------------
# variants the reference's pytest never covered: non-causal, chunk-visible, FDA, D=128, fp32
# ---------------------------------------------------------------------------
VARIANTS = [
    # B, T, H, D, L, G, mode, chunk_tokens, dtype
    (2, 197, 3, 64, 12, 1, "noncausal", 0, torch.bfloat16),
    (2, 197, 1, 64, 11, 4, "noncausal", 0, torch.float16),
    (1, 130, 2, 128, 5, 2, "noncausal", 0, torch.bfloat16),
    (1, 64, 2, 64, 0, 2, "noncausal", 0, torch.float16),
    (1, 300, 2, 128, 6, 4, "chunk_visible", 16, torch.bfloat16),
    (2, 129, 2, 64, 3, 1, "chunk_visible", 64, torch.float16),
    (1, 257, 1, 128, 24, 4, "chunk_visible", 16, torch.bfloat16),
    (1, 100, 2, 64, 7, 2, "chunk_visible", 1, torch.bfloat16),
    (1, 90, 2, 64, 0, 2, "chunk_visible", 32, torch.bfloat16),
    (2, 197, 3, 64, 12, 1, "depth_only", 0, torch.bfloat16),
    (1, 100, 2, 128, 7, 4, "depth_only", 0, torch.float16),
    (1, 33, 1, 64, 72, 2, "depth_only", 0, torch.float16),
    (1, 1, 1, 128, 1, 1, "depth_only", 0, torch.bfloat16),
    (2, 260, 2, 128, 8, 4, "causal", 0, torch.bfloat16),
    (1, 128, 2, 64, 72, 2, "causal", 0, torch.float16),
    (1, 513, 1, 128, 3, 8, "causal", 0, torch.float16),
    (1, 3, 2, 128, 2, 16, "causal", 0, torch.bfloat16),
    (1, 256, 4, 64, 4, 1, "causal", 0, torch.float32),
    (1, 70, 2, 32, 3, 2, "noncausal", 0, torch.float32),
    (1, 50, 2, 64, 3, 2, "depth_only", 0, torch.float32),
    (1, 100, 2, 32, 3, 2, "chunk_visible", 8, torch.float32),
    (1, 100, 2, 96, 3, 2, "causal", 0, torch.bfloat16),
    (1, 60, 1, 256, 2, 1, "causal", 0, torch.float16),
    # head dims below the matrix kernels' tile widths (64, 128): zero-padded inside the kernels
    (2, 70, 2, 32, 3, 2, "causal", 0, torch.bfloat16),
    (1, 150, 2, 96, 5, 4, "chunk_visible", 16, torch.float16),
    (2, 64, 3, 96, 4, 1, "depth_only", 0, torch.bfloat16),
    (1, 100, 2, 72, 2, 2, "noncausal", 0, torch.bfloat16),
    (1, 90, 1, 8, 2, 2, "causal", 0, torch.float16),
    (1, 200, 2, 120, 3, 4, "causal", 0, torch.bfloat16),
    (2, 45, 2, 36, 3, 2, "causal", 0, torch.bfloat16),     # rows of 72 bytes: not 16-byte aligned
    (1, 40, 3, 100, 2, 1, "noncausal", 0, torch.float16),  # rows of 200 bytes
    # head dims above 128: the 256-wide tiles (16 query rows per wave), zero-padded for 136..248
    (1, 300, 2, 256, 5, 2, "causal", 0, torch.bfloat16),
    (1, 260, 2, 256, 0, 4, "causal", 0, torch.bfloat16),
    (2, 130, 2, 192, 6, 4, "chunk_visible", 16, torch.float16),
    (1, 700, 1, 256, 3, 2, "chunk_visible", 64, torch.bfloat16),
    (1, 197, 3, 160, 12, 1, "noncausal", 0, torch.bfloat16),
    (1, 100, 2, 256, 7, 4, "depth_only", 0, torch.float16),
    (1, 150, 1, 136, 2, 2, "causal", 0, torch.float16),
    # 64-wide tiles outside chunk-visible mode: the dQ kernel forms the depth gradients when the query group divides
    # a wave's 32 rows (groups of 8, 16, 32; the throughput launch shape), the depth-column kernel otherwise (3, 5)
    (1, 77, 2, 64, 5, 8, "causal", 0, torch.bfloat16),
    (1, 300, 1, 64, 2, 16, "depth_only", 0, torch.bfloat16),
    (1, 40, 1, 64, 3, 32, "noncausal", 0, torch.float16),
    (2, 90, 2, 64, 4, 3, "causal", 0, torch.bfloat16),
    (1, 50, 1, 48, 6, 5, "depth_only", 0, torch.float16),
    (8, 520, 8, 64, 1, 4, "causal", 0, torch.bfloat16),
    # 64-wide tiles with at least three sequence column tiles per compute unit and more than 512 query rows: the
    # sequence dK/dV of these go to the four-wave kernel by the size of the grid, not by their length
    (12, 1024, 8, 64, 2, 2, "causal", 0, torch.bfloat16),
    (6, 1100, 16, 48, 0, 1, "noncausal", 0, torch.float16),
]


@pytest.mark.parametrize("case", VARIANTS, ids=lambda c: f"{c[6]}-T{c[1]}-D{c[3]}-L{c[4]}-G{c[5]}-{str(c[8])[6:]}")
def test_variants(gpu_device, case):
    B, T, H, D, L, G, mode, cb, dtype = case
    say(f"[variant] {case}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=7, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, mode, cb)
    got = run_hip(to_dev(inp, gpu_device), sc, G, mode, cb)
    compare_all(got, ref, dtype, str(case))


@pytest.mark.parametrize("case", [
    # (B, T, H, D, L, G, mode, chunk tokens, compute type)
    (1, 256, 4, 64, 4, 2, "causal", 0, "fp16"),          # the fp32 plumbing configuration of the benchmark list
    (2, 197, 3, 64, 12, 1, "noncausal", 0, "fp16"),
    (1, 300, 2, 128, 6, 4, "chunk_visible", 16, "bf16"),
    (1, 100, 2, 96, 3, 2, "depth_only", 0, "fp16"),
])
def test_fp32_inputs_through_the_matrix_kernels(gpu_device, case):
    """``set_fp32_compute("fp16" | "bf16")``: fp32 tensors are rounded to the 16-bit type, run on the matrix kernels and
    come back as fp32 -- for fp16 the same operand precision as the reference's fp32 path (tl.dot's default input
    precision keeps a 10-bit mantissa, moda_v14.py:188, 209).  Checked against the oracle on the UNROUNDED fp32 inputs
    at the 16-bit type's tolerance; the default setting stays exact fp32 (every other fp32 case of this file)."""
    import moda_amd
    from moda_amd import ops

    B, T, H, D, L, G, mode, cb, how = case
    say(f"CASE fp32-compute {case}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=41, dtype=torch.float32, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, mode, cb)
    previous = moda_amd.set_fp32_compute(how)
    try:
        assert previous == "fp32"
        got = run_hip(to_dev(inp, gpu_device), sc, G, mode, cb)
        # accumulate flag: fp32 buffers that already hold something
        dev = to_dev(inp, gpu_device)
        m = MODE_ID[mode]
        o, lse = ops._raw_fwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], sc, G, cb)
        held = tuple(None if dev[n] is None else torch.ones_like(dev[n]) for n in ("q", "k", "v", "kd", "vd"))
        ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], o, lse, dev["do"], sc, G, cb, out=held,
                     accumulate_depth=True)
    finally:
        assert moda_amd.set_fp32_compute(previous) == how
    narrow = torch.float16 if how == "fp16" else torch.bfloat16
    for name, x in got.items():
        assert x is None or x.dtype == torch.float32, name
    compare_all(got, ref, narrow, f"fp32 via {how} {case}")
    assert torch.equal(held[0], got["dq"]) and (held[1] is None or torch.equal(held[1], got["dk"]))
    assert torch.equal(held[3], got["dkd"] + 1.0) and torch.equal(held[4], got["dvd"] + 1.0)


def test_golden_fixture(gpu_device):
    """Committed fixture (tests/golden/moda_small.npz) against the HIP kernels in fp32 and bf16."""
    import os

    import numpy as np

    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "moda_small.npz"))
    for mode, cb in (("causal", 0), ("noncausal", 0), ("chunk_visible", 4), ("depth_only", 0)):
        B, T, H, D, L, G, seed = (int(x) for x in z[f"{mode}_meta"])
        for dtype in (torch.float32, torch.bfloat16):
            say(f"[golden] {mode} {dtype}")
            inp = oracle.make_inputs(B, T, H, D, L, G, seed=seed, dtype=torch.float32, std=0.5,
                                     depth_only=(mode == "depth_only"))
            if dtype != torch.float32:
                # the fixture was computed from the fp32 inputs; rounding them to bf16 moves the answer by more
                # than the output tolerance, so only the forward outputs are compared, with a widened bound
                inp = {k: (None if v is None else v.to(dtype)) for k, v in inp.items()}
            got = run_hip(to_dev(inp, gpu_device), D ** -0.5, G, mode, cb)
            if dtype == torch.float32:
                for n in ("o", "lse", "dq", "dk", "dv", "dkd", "dvd"):
                    if f"{mode}_{n}" in z:
                        check(n, got[n], torch.from_numpy(z[f"{mode}_{n}"]), dtype, f"golden {mode}")
            else:
                err = (got["o"].float().cpu() - torch.from_numpy(z[f"{mode}_o"])).abs().max().item()
                assert err < 3e-2, (mode, err)


# ---------------------------------------------------------------------------
# the five benchmark configurations (c1 .. c5)
# ---------------------------------------------------------------------------
def test_config_c1_fp32(gpu_device):
    """B1 T256 H4 D64 L4 fp32, q pre-scaled by D**-0.5 and scale=1 -- on the GPU in fp32."""
    inp = oracle.make_inputs(1, 256, 4, 64, 4, 1, seed=0, dtype=torch.float32, prescale_q=True)
    ref = oracle.moda_dense_fwd_bwd(inp, 1.0, 1, "causal")
    got = run_hip(to_dev(inp, gpu_device), 1.0, 1, "causal")
    compare_all(got, ref, torch.float32, "c1", plain_atol=2e-4)
    # literal row loops on a slice of rows as a second opinion
    o_rows, lse_rows = oracle.moda_rows(inp["q"][:, :40], inp["k"][:, :40], inp["v"][:, :40], inp["kd"][:, :160],
                                        inp["vd"][:, :160], 1.0, 1, "causal")
    check("o", got["o"][:, :40], o_rows, torch.float32, "c1 rows")
    check("lse", got["lse"][:, :40], lse_rows, torch.float32, "c1 rows")


def _blockwise_on_gpu(inp_dev, sc, G, mode, cb, dtype, block_rows=4096):
    return oracle.moda_blockwise_fwd_bwd(inp_dev, sc, G, mode, cb, block_rows=block_rows, dtype=torch.float32,
                                         o_round_dtype=dtype)


def test_blockwise_oracle_on_gpu_matches_dense(gpu_device):
    """The tiled oracle form used for the large configs, run on the GPU, equals the dense CPU form."""
    inp = oracle.make_inputs(1, 300, 2, 128, 6, 4, seed=5, dtype=torch.bfloat16, std=0.5)
    for mode, cb in (("causal", 0), ("chunk_visible", 16), ("noncausal", 0)):
        ref = oracle.moda_dense_fwd_bwd(inp, 0.1, 4, mode, cb)
        blk = oracle.moda_blockwise_fwd_bwd(to_dev(inp, gpu_device), 0.1, 4, mode, cb, block_rows=256)
        for n in ("o", "lse", "dq", "dk", "dv", "dkd", "dvd"):
            assert torch.allclose(blk[n].cpu(), ref[n], atol=2e-5, rtol=1e-4), (mode, n)


def test_config_c2(gpu_device):
    """moda_v14 causal bf16 B2 T4096 Hq16 Hkv4 D128 L8: all tensors against the tiled oracle."""
    B, T, H, D, L, G = 2, 4096, 4, 128, 8, 4
    say("[c2] generating inputs")
    inp = to_dev(oracle.make_inputs(B, T, H, D, L, G, seed=0, dtype=torch.bfloat16, std=0.5), gpu_device)
    sc = D ** -0.5
    got = run_hip(inp, sc, G, "causal")
    say("[c2] oracle")
    ref = _blockwise_on_gpu(inp, sc, G, "causal", 0, torch.bfloat16)
    compare_all(got, ref, torch.bfloat16, "c2", plain_atol=2e-2)
    # row subsample against the dense form evaluated on the CPU
    rows = torch.tensor([0, 1, 5, 4095, 8191, 8192, 12345, 16383])
    cpu = {k: (None if v is None else v.cpu()) for k, v in inp.items()}
    sub = oracle.moda_rows_subset(cpu, rows, sc, G, "causal")
    check("o", got["o"][:, rows], sub["o"], torch.bfloat16, "c2 rows")
    check("lse", got["lse"][:, rows], sub["lse"], torch.bfloat16, "c2 rows")
    check("dq", got["dq"][:, rows], sub["dq"], torch.bfloat16, "c2 rows")


def _sum_invariants(inp, got, what):
    """Size-independent properties: rows of P sum to one => sum dV + sum dVd == sum dO;
    bilinearity => <q,dq> == <k,dk> + <kd,dkd>."""
    f = lambda x: x.double()
    tot = torch.zeros_like(f(inp["do"]).sum(1))
    mag = torch.zeros_like(tot)
    for n in ("dv", "dvd"):
        if got[n] is not None:
            tot += f(got[n]).sum(1)
            mag += f(got[n]).abs().sum(1)
    want = f(inp["do"]).sum(1)
    # every stored gradient carries a relative rounding error of <= 2**-9
    assert ((tot - want).abs() <= 2.0 ** -8 * mag + 1e-3).all(), f"{what}: sum dV invariant"
    lhs = (f(inp["q"]) * f(got["dq"])).sum()
    rhs = sum((f(inp[n]) * f(got["d" + n])).sum() for n in ("k", "kd") if inp[n] is not None)
    scale = sum((f(inp[n]) * f(got["d" + n])).abs().sum() for n in ("q", "k", "kd") if inp[n] is not None)
    assert abs(lhs - rhs) <= 2.0 ** -8 * scale + 1e-3, f"{what}: <q,dq> invariant {lhs} vs {rhs}"


def test_config_c3_chunk_visible(gpu_device):
    """moda_v16 chunk-visible bf16 B1 T16384 Hq16 Hkv4 D128 L24 C64."""
    B, T, H, D, L, G, cb = 1, 16384, 4, 128, 24, 4, 16
    say("[c3] generating inputs")
    inp = to_dev(oracle.make_inputs(B, T, H, D, L, G, seed=0, dtype=torch.bfloat16, std=0.5), gpu_device)
    sc = D ** -0.5
    got = run_hip(inp, sc, G, "chunk_visible", cb)
    torch.cuda.synchronize()
    say("[c3] oracle")
    ref = _blockwise_on_gpu(inp, sc, G, "chunk_visible", cb, torch.bfloat16)
    compare_all(got, ref, torch.bfloat16, "c3", plain_atol=2e-2)
    _sum_invariants(inp, got, "c3")
    rows = torch.tensor([0, 63, 64, 65, 127, 32768, 65535], device=gpu_device)
    sub = oracle.moda_rows_subset(inp, rows, sc, G, "chunk_visible", cb)
    check("o", got["o"][:, rows], sub["o"], torch.bfloat16, "c3 rows")
    check("lse", got["lse"][:, rows], sub["lse"], torch.bfloat16, "c3 rows")
    check("dq", got["dq"][:, rows], sub["dq"], torch.bfloat16, "c3 rows")


def test_config_c4_headline_and_plain_twin(gpu_device):
    """Headline: causal bf16 B1 T65536 Hq16 Hkv4 D128 L24, and the plain causal twin of the same build."""
    from moda_amd import ops

    B, T, H, D, L, G = 1, 65536, 4, 128, 24, 4
    say("[c4] generating inputs")
    inp = to_dev(oracle.make_inputs(B, T, H, D, L, G, seed=0, dtype=torch.bfloat16, std=0.5), gpu_device)
    sc = D ** -0.5
    got = run_hip(inp, sc, G, "causal")
    torch.cuda.synchronize()
    say("[c4] invariants")
    _sum_invariants(inp, got, "c4")
    say("[c4] oracle")
    ref = _blockwise_on_gpu(inp, sc, G, "causal", 0, torch.bfloat16, block_rows=8192)
    compare_all(got, ref, torch.bfloat16, "c4", plain_atol=2e-2)
    del ref
    rows = torch.tensor([0, 3, 4, 131071, 131072, 262143], device=gpu_device)
    sub = oracle.moda_rows_subset(inp, rows, sc, G, "causal")
    check("o", got["o"][:, rows], sub["o"], torch.bfloat16, "c4 rows")
    check("lse", got["lse"][:, rows], sub["lse"], torch.bfloat16, "c4 rows")
    check("dq", got["dq"][:, rows], sub["dq"], torch.bfloat16, "c4 rows")
    # plain twin: the same q rows viewed as [B, T, G*Hkv, D] would be group-major; the twin uses kv-major
    # head order (hq // G), so compare it with the folded kernel run WITHOUT depth on re-ordered heads.
    say("[c4] plain twin")
    q_plain = inp["q"].view(B, T, G, H, D).permute(0, 1, 3, 2, 4).reshape(B, T, H * G, D).contiguous()
    do_plain = inp["do"].view(B, T, G, H, D).permute(0, 1, 3, 2, 4).reshape(B, T, H * G, D).contiguous()
    o_p, lse_p = ops.parallel_attn_fwd(q_plain, inp["k"], inp["v"], None, sc)
    dq_p, dk_p, dv_p, _ = ops.parallel_attn_bwd(q_plain, inp["k"], inp["v"], o_p, None, lse_p, do_plain, sc)
    nod = dict(inp)
    nod["kd"] = nod["vd"] = None
    ref2 = _blockwise_on_gpu(nod, sc, G, "causal", 0, torch.bfloat16, block_rows=8192)
    unfold = lambda x: x.view(B, T, H, G, -1).permute(0, 1, 3, 2, 4).reshape(B, T * G, H, -1)
    check("o", unfold(o_p), ref2["o"], torch.bfloat16, "twin")
    check("lse", unfold(lse_p.unsqueeze(-1)).squeeze(-1), ref2["lse"], torch.bfloat16, "twin")
    check("dq", unfold(dq_p), ref2["dq"], torch.bfloat16, "twin")
    check("dk", dk_p, ref2["dk"], torch.bfloat16, "twin")
    check("dv", dv_p, ref2["dv"], torch.bfloat16, "twin")


def test_config_c5_deit_noncausal_and_fda(gpu_device):
    """DeiT-S shape bf16 B64 T197 H6 D64 L12: non-causal MoDA and FDA on the same tensors."""
    B, T, H, D, L, G = 64, 197, 6, 64, 12, 1
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=0, dtype=torch.bfloat16, std=0.5)
    dev = to_dev(inp, gpu_device)
    sc = D ** -0.5
    got = run_hip(dev, sc, G, "noncausal")
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, "noncausal")
    compare_all(got, ref, torch.bfloat16, "c5 noncausal", plain_atol=2e-2)
    fda_in = dict(dev)
    fda_in["k"] = fda_in["v"] = None
    got = run_hip(fda_in, sc, G, "depth_only")
    cpu_in = dict(inp)
    cpu_in["k"] = cpu_in["v"] = None
    ref = oracle.moda_dense_fwd_bwd(cpu_in, sc, G, "depth_only")
    compare_all(got, ref, torch.bfloat16, "c5 fda", plain_atol=2e-2)


# ---------------------------------------------------------------------------
# operator interface: autograd, LSE, layouts, dtypes
# ---------------------------------------------------------------------------
def test_autograd_interface_and_lse(gpu_device):
    import moda_amd

    B, T, H, D, L, G = 2, 96, 2, 64, 5, 2
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=11, dtype=torch.float16, std=0.5)
    ref = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, "causal")
    dev = to_dev(inp, gpu_device)
    leaves = {n: dev[n].clone().requires_grad_(True) for n in ("q", "k", "v", "kd", "vd")}
    o, lse = moda_amd.parallel_moda(leaves["q"], leaves["k"], leaves["v"], cached_k=leaves["kd"],
                                    cached_v=leaves["vd"], moda_group_num=G, need_lse=True)
    assert o.dtype == torch.float16 and lse.dtype == torch.float32 and not lse.requires_grad
    (o * dev["do"]).sum().backward()
    got = {"o": o, "lse": lse, "dq": leaves["q"].grad, "dk": leaves["k"].grad, "dv": leaves["v"].grad,
           "dkd": leaves["kd"].grad, "dvd": leaves["vd"].grad}
    compare_all(got, ref, torch.float16, "autograd")
    # without depth: cached grads are None, o only
    o2 = moda_amd.parallel_moda(dev["q"], dev["k"], dev["v"], moda_group_num=G)
    assert isinstance(o2, torch.Tensor)
    # head_first layout
    o3 = moda_amd.parallel_moda(dev["q"].transpose(1, 2), dev["k"].transpose(1, 2), dev["v"].transpose(1, 2),
                                cached_k=dev["kd"].transpose(1, 2), cached_v=dev["vd"].transpose(1, 2),
                                moda_group_num=G, head_first=True)
    assert torch.equal(o3, o.detach())


def test_chunk_visible_and_fda_autograd(gpu_device):
    import moda_amd

    B, T, H, D, L, G = 1, 150, 2, 64, 3, 4
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=13, dtype=torch.bfloat16, std=0.5)
    dev = to_dev(inp, gpu_device)
    leaves = {n: dev[n].clone().requires_grad_(True) for n in ("q", "k", "v", "kd", "vd")}
    o, lse = moda_amd.parallel_moda_chunk_visible(leaves["q"], leaves["k"], leaves["v"], cached_k=leaves["kd"],
                                                  cached_v=leaves["vd"], moda_group_num=G, need_lse=True)
    (o * dev["do"]).sum().backward()
    ref = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, "chunk_visible", 64 // G)
    got = {"o": o, "lse": lse, "dq": leaves["q"].grad, "dk": leaves["k"].grad, "dv": leaves["v"].grad,
           "dkd": leaves["kd"].grad, "dvd": leaves["vd"].grad}
    compare_all(got, ref, torch.bfloat16, "chunk-visible autograd")

    leaves = {n: dev[n].clone().requires_grad_(True) for n in ("q", "kd", "vd")}
    o = moda_amd.parallel_fda(leaves["q"], cached_k=leaves["kd"], cached_v=leaves["vd"], moda_group_num=G)
    (o * dev["do"]).sum().backward()
    fin = dict(inp)
    fin["k"] = fin["v"] = None
    ref = oracle.moda_dense_fwd_bwd(fin, D ** -0.5, G, "depth_only")
    check("o", o, ref["o"], torch.bfloat16, "fda")
    check("dq", leaves["q"].grad, ref["dq"], torch.bfloat16, "fda")
    check("dkd", leaves["kd"].grad, ref["dkd"], torch.bfloat16, "fda")
    check("dvd", leaves["vd"].grad, ref["dvd"], torch.bfloat16, "fda")


def test_deit_style_caller(gpu_device):
    """The in-repo caller's pattern (vision_tasks/deit/models.py:244-267): k, v are strided slices of a fused
    kv projection, fp16 under autocast, is_causal=False, depth cache built from earlier layers."""
    import moda_amd

    B, N, G, Hkv, D, nl = 4, 197, 4, 1, 64, 3
    gen = torch.Generator().manual_seed(3)
    q = (torch.randn(B, N * G, Hkv, D, generator=gen) * 0.5).half().to(gpu_device).requires_grad_(True)
    kv = (torch.randn(B, N, 2, Hkv, D, generator=gen) * 0.5).half().to(gpu_device).requires_grad_(True)
    prev = [((torch.randn(B, N, Hkv, D, generator=gen) * 0.5).half().to(gpu_device).requires_grad_(True),
             (torch.randn(B, N, Hkv, D, generator=gen) * 0.5).half().to(gpu_device).requires_grad_(True))
            for _ in range(nl)]
    k, v = kv[:, :, 0], kv[:, :, 1]
    assert not k.is_contiguous()
    dk_cache, dv_cache = moda_amd.build_depth_cache(prev)
    o = moda_amd.parallel_moda(q=q, k=k, v=v, g=None, scale=D ** -0.5, cu_seqlens=None, cached_k=dk_cache,
                               cached_v=dv_cache, moda_group_num=G, is_causal=False, head_first=False,
                               warn_shape=False)
    do = (torch.randn(B, N * G, Hkv, D, generator=gen)).half().to(gpu_device)
    (o * do).sum().backward()
    # oracle with the reference's own cache construction
    kd_ref = oracle.depth_cache_ref([p[0].detach().cpu() for p in prev])
    vd_ref = oracle.depth_cache_ref([p[1].detach().cpu() for p in prev])
    inp = {"q": q.detach().cpu(), "k": k.detach().cpu(), "v": v.detach().cpu(), "kd": kd_ref, "vd": vd_ref,
           "do": do.cpu()}
    ref = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, "noncausal")
    check("o", o, ref["o"], torch.float16, "deit")
    check("dq", q.grad, ref["dq"], torch.float16, "deit")
    check("dk", kv.grad[:, :, 0], ref["dk"], torch.float16, "deit")
    check("dv", kv.grad[:, :, 1], ref["dv"], torch.float16, "deit")
    dkd_layers = oracle.depth_cache_grad_ref(ref["dkd"], nl)
    dvd_layers = oracle.depth_cache_grad_ref(ref["dvd"], nl)
    for l in range(nl):
        check("dkd", prev[l][0].grad, dkd_layers[l], torch.float16, f"deit layer {l}")
        check("dvd", prev[l][1].grad, dvd_layers[l], torch.float16, f"deit layer {l}")


def test_deit_style_caller_under_autocast(gpu_device):
    """The reference's training loop runs the model under torch.cuda.amp.autocast() with fp32 parameters
    (vision_tasks/deit/engine.py:46-47): the projections come out in fp16 inside the autocast region, the
    operator's autograd Function (custom_fwd / custom_bwd) sees fp16 tensors, and the parameter gradients
    come back in fp32."""
    import moda_amd

    torch.manual_seed(5)
    B, N, dim, heads, kv_heads = 3, 197, 256, 4, 1
    attn = moda_amd.MoDAAttention(dim, heads, kv_heads, qkv_bias=True).to(gpu_device)  # fp32 parameters
    D, G = attn.head_dim, attn.moda_group_num
    x = (0.5 * torch.randn(B, N, dim, device=gpu_device)).requires_grad_(True)
    prev = [(0.5 * torch.randn(B, N, kv_heads, D, device=gpu_device)).requires_grad_(True) for _ in range(4)]
    w = torch.randn(B, N, dim, device=gpu_device)
    seen = {}
    real = moda_amd.modules.parallel_moda

    def spy(**kw):
        seen["dtypes"] = {n: kw[n].dtype for n in ("q", "k", "v", "cached_k", "cached_v")}
        seen["args"] = {n: kw[n].detach().clone() for n in ("q", "k", "v", "cached_k", "cached_v")}
        o = real(**kw)
        o.retain_grad()
        seen["o"] = o
        return o

    moda_amd.modules.parallel_moda = spy
    try:
        with torch.autocast("cuda", dtype=torch.float16):
            dk_cache = moda_amd.stack_depth([p.half() for p in prev[:2]])
            dv_cache = moda_amd.stack_depth([p.half() for p in prev[2:]])
            y, k, v = attn(x, depth_k=dk_cache, depth_v=dv_cache)
            loss = (y.float() * w).sum()
        loss.backward()
    finally:
        moda_amd.modules.parallel_moda = real
    assert all(dt == torch.float16 for dt in seen["dtypes"].values()), seen["dtypes"]
    assert attn.q.weight.grad.dtype == torch.float32 and x.grad.dtype == torch.float32
    assert all(p.grad is not None and p.grad.abs().max() > 0 for p in prev)
    # the operator call itself against the oracle on the very tensors it received
    a = seen["args"]
    inp = {"q": a["q"].cpu(), "k": a["k"].cpu(), "v": a["v"].cpu(), "kd": a["cached_k"].cpu(),
           "vd": a["cached_v"].cpu(), "do": seen["o"].grad.cpu()}
    ref = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, "noncausal")
    check("o", seen["o"], ref["o"], torch.float16, "autocast")
    # the gradient that reached the depth layers (fp32 leaves) is the slot-wise split of dkd / dvd
    for l, (gk, gv) in enumerate(zip(oracle.depth_cache_grad_ref(ref["dkd"], 2), oracle.depth_cache_grad_ref(ref["dvd"], 2))):
        check("dkd", prev[l].grad, gk, torch.float16, f"autocast layer {l}")
        check("dvd", prev[2 + l].grad, gv, torch.float16, f"autocast layer {l}")


def test_integration_stub_as_documented(gpu_device, monkeypatch):
    """The repository's integration notes show the ctypes binding a maintainer of the reference would put in place
    of the bodies of parallel_moda_fwd / parallel_moda_bwd (moda_v14.py:381-522, 1470-1842).  This runs that very
    text (only ctypes and torch; the library is found next to the package instead of on the loader path) and holds
    its results to the parity bar."""
    import ctypes
    import os
    import re

    import moda_amd

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    block = re.search(r"```python\n(import ctypes, torch.*?)```", text, flags=re.S).group(1)
    real_cdll = ctypes.CDLL
    monkeypatch.setattr(ctypes, "CDLL", lambda name, *a, **kw: real_cdll(
        os.path.join(os.path.dirname(moda_amd.__file__), name) if name == "libmoda_hip.so" else name, *a, **kw))
    ns = {}
    exec(compile(block, "integration-notes-stub", "exec"), ns)
    for (B, T, H, D, L, G, causal, dtype) in [(2, 150, 2, 64, 5, 2, True, torch.bfloat16),
                                              (1, 197, 3, 128, 4, 1, False, torch.float16),
                                              (1, 90, 2, 128, 0, 4, True, torch.bfloat16)]:
        say(f"[integration stub] B{B} T{T} H{H} D{D} L{L} G{G} causal={causal} {dtype}")
        inp = oracle.make_inputs(B, T, H, D, L, G, seed=71, dtype=dtype, std=0.5)
        sc = D ** -0.5
        ref = oracle.moda_dense_fwd_bwd(inp, sc, G, "causal" if causal else "noncausal")
        d = to_dev(inp, gpu_device)
        o, lse = ns["parallel_moda_fwd"](d["q"], d["k"], d["v"], None, sc, cached_k=d["kd"], cached_v=d["vd"],
                                         moda_group_num=G, is_causal=causal)
        dq, dk, dv, _, dkd, dvd = ns["parallel_moda_bwd"](d["q"], d["k"], d["v"], o, None, lse, d["do"], sc,
                                                          cached_k=d["kd"], cached_v=d["vd"], moda_group_num=G,
                                                          is_causal=causal)
        compare_all({"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}, ref, dtype,
                    "integration stub")


def test_plain_gqa_attention(gpu_device):
    import moda_amd

    B, T, Hkv, G, D = 2, 333, 2, 4, 128
    inp = oracle.make_inputs(B, T, Hkv, D, 0, G, seed=17, dtype=torch.bfloat16, std=0.5, Hq=Hkv * G)
    leaf = {n: inp[n].float().clone().requires_grad_(True) for n in ("q", "k", "v")}
    o_ref, lse_ref = oracle.plain_gqa_dense(leaf["q"], leaf["k"], leaf["v"])
    (o_ref * inp["do"].float()).sum().backward()
    dev = to_dev(inp, gpu_device)
    dl = {n: dev[n].clone().requires_grad_(True) for n in ("q", "k", "v")}
    o = moda_amd.parallel_attn(dl["q"], dl["k"], dl["v"])
    (o * dev["do"]).sum().backward()
    check("o", o, o_ref, torch.bfloat16, "plain")
    for n in ("q", "k", "v"):
        check("d" + n, dl[n].grad, leaf[n].grad, torch.bfloat16, "plain")
    _, lse = moda_amd.parallel_attn_fwd(dev["q"], dev["k"], dev["v"])
    check("lse", lse, lse_ref, torch.bfloat16, "plain")


def test_bitwise_determinism(gpu_device):
    inp = to_dev(oracle.make_inputs(2, 700, 2, 128, 6, 4, seed=19, dtype=torch.bfloat16, std=0.5), gpu_device)
    a = run_hip(inp, 0.1, 4, "causal")
    b = run_hip(inp, 0.1, 4, "causal")
    for n in a:
        assert torch.equal(a[n], b[n]), n


def test_slices_wider_than_32bit_offsets(gpu_device):
    """K/V and depth K/V read in place from views whose (batch, head) slice spans more bytes than a
    32-bit buffer offset reaches: results must equal those of compact copies bit for bit."""
    B, T, H, D, L, G = 1, 4096, 1, 64, 2, 2
    inp = to_dev(oracle.make_inputs(B, T, H, D, L, G, seed=23, dtype=torch.bfloat16, std=0.5), gpu_device)
    row = 1 << 19  # elements between rows: 1 MiB, so 4096 rows span 4 GiB and the depth rows 8 GiB

    def spread(x):
        rows = x.shape[1]
        buf = torch.empty(rows * row, dtype=x.dtype, device=x.device)
        view = buf.as_strided((B, rows, H, D), (rows * row, row, D, 1))
        view.copy_(x)
        return view

    wide = dict(inp)
    for n in ("k", "v", "kd", "vd"):
        wide[n] = spread(inp[n])
        assert wide[n].stride(1) * wide[n].shape[1] * 2 >= (1 << 32)
    say("CASE wide-slices")
    a = run_hip(inp, D ** -0.5, G, "causal")
    b = run_hip(wide, D ** -0.5, G, "causal")
    for n in a:
        assert torch.equal(a[n], b[n]), n
    rows = torch.tensor([0, 1, 4095 * G, T * G - 1])
    cpu = {k: (None if v is None else v.cpu()) for k, v in inp.items()}
    ref = oracle.moda_rows_subset(cpu, rows, D ** -0.5, G, "causal")
    check("o", b["o"][:, rows.to(gpu_device)], ref["o"], torch.bfloat16, "wide-slices")
    check("dq", b["dq"][:, rows.to(gpu_device)], ref["dq"], torch.bfloat16, "wide-slices")
    # the same views as a packed variable-length batch
    from moda_amd import ops

    say("CASE wide-slices packed")
    packed = ops._packed(torch.tensor([0, 1000, 1001, T], device=gpu_device), inp["q"], G)

    def run_packed(x):
        o, lse = ops._raw_fwd(0, x["q"], x["k"], x["v"], x["kd"], x["vd"], D ** -0.5, G, packed=packed)
        return (o, lse) + tuple(ops._raw_bwd(0, x["q"], x["k"], x["v"], x["kd"], x["vd"], o, lse, x["do"], D ** -0.5, G,
                                             packed=packed))

    for i, (x, y) in enumerate(zip(run_packed(inp), run_packed(wide))):
        assert torch.equal(x, y), i


@pytest.mark.parametrize("case", [
    # (B, T, H, D, L, valid, G, mode, dtype, chunk tokens)
    (2, 150, 2, 64, 5, 3, 2, "causal", torch.bfloat16, 0),
    (1, 333, 2, 128, 6, 1, 4, "causal", torch.bfloat16, 0),
    (2, 197, 3, 64, 12, 7, 1, "noncausal", torch.float16, 0),
    (2, 97, 2, 128, 4, 4, 1, "causal", torch.bfloat16, 0),
    (2, 130, 2, 64, 9, 2, 2, "depth_only", torch.bfloat16, 0),
    (1, 70, 2, 96, 5, 2, 2, "causal", torch.bfloat16, 0),    # head dim zero-padded to 128
    (1, 70, 2, 36, 5, 2, 2, "causal", torch.bfloat16, 0),    # vector-ALU kernels (head dim not a multiple of 8)
    (1, 60, 2, 64, 3, 2, 1, "causal", torch.float32, 0),     # vector-ALU kernels (fp32)
    (1, 300, 2, 256, 5, 2, 2, "causal", torch.bfloat16, 0),  # 256-wide tiles: depth columns through the ring
    (3, 2100, 1, 128, 3, 2, 2, "causal", torch.bfloat16, 0),  # the throughput launch shape
    # chunk-visible: chunks within one query tile (the waves' own depth tiles, the chunk kernel), above it (ring
    # depth tiles, depth column tiles), on the 256-wide tiles, on the vector-ALU kernels
    (1, 300, 2, 128, 6, 4, 4, "chunk_visible", torch.bfloat16, 16),
    (2, 130, 1, 64, 7, 1, 2, "chunk_visible", torch.float16, 8),
    (1, 260, 1, 64, 3, 2, 4, "chunk_visible", torch.bfloat16, 40),
    (1, 400, 2, 128, 5, 3, 4, "chunk_visible", torch.bfloat16, 32),
    (1, 200, 2, 192, 5, 3, 2, "chunk_visible", torch.float16, 16),
    (1, 90, 2, 32, 4, 3, 2, "chunk_visible", torch.float32, 8),
])
def test_partially_filled_depth_stream(gpu_device, case):
    """depth_valid = v on the L-slot tensors == the compacted [B, T*v, H, D] tensors (the oracle's
    definition).  The unused slots hold NaN, Inf and huge finite values -- an uninitialised cache -- which
    must neither reach any output nor be read; their gradients must come out exactly zero."""
    from moda_amd import ops

    B, T, H, D, L, valid, G, mode, dtype, cb = case
    say(f"CASE partial-depth {case}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=29, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    junk = torch.Generator().manual_seed(5)
    for n in ("kd", "vd"):
        x = inp[n].reshape(B, T, L, H, D)
        fill = 30.0 * torch.randn(x[:, :, valid:].shape, generator=junk)
        pick = torch.rand(fill.shape, generator=junk)
        fill[pick < 0.3] = float("nan")
        fill[(pick >= 0.3) & (pick < 0.45)] = float("inf")
        fill[(pick >= 0.45) & (pick < 0.6)] = float("-inf")
        x[:, :, valid:] = fill.to(dtype)
    comp = dict(inp)
    comp["kd"] = oracle.compact_depth(inp["kd"], T, valid).contiguous()
    comp["vd"] = oracle.compact_depth(inp["vd"], T, valid).contiguous()
    scale = D ** -0.5
    ref = oracle.moda_dense_fwd_bwd(comp, scale, G, mode, cb)
    ref["dkd"] = oracle.scatter_depth_grad(ref["dkd"], T, L)
    ref["dvd"] = oracle.scatter_depth_grad(ref["dvd"], T, L)
    dev = to_dev(inp, gpu_device)
    m = MODE_ID[mode]
    o, lse = ops._raw_fwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], scale, G, cb, depth_valid=valid)
    # the gradient buffers start as NaN: every element must be written
    out = tuple(None if dev[n] is None else torch.full_like(dev[n], float("nan")) for n in ("q", "k", "v", "kd", "vd"))
    dq, dk, dv, dkd, dvd = ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], o, lse, dev["do"], scale,
                                        G, cb, depth_valid=valid, out=out)
    got = {"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}
    compare_all(got, ref, dtype, f"partial-depth {case}")
    for n in ("dkd", "dvd"):
        unused = got[n].reshape(B, T, L, H, D)[:, :, valid:]
        assert unused.numel() == 0 or unused.float().abs().max().item() == 0.0, n


def test_depth_cache_append_in_place(gpu_device):
    """DepthCache.append + depth_valid reproduces, layer by layer, what the rebuilt compact cache gives
    (vision_tasks/deit/models.py:383-387 rebuilds it for every layer)."""
    import moda_amd

    B, T, H, D, Lmax, G = 2, 64, 2, 64, 4, 2
    gen = torch.Generator().manual_seed(31)
    q = (0.5 * torch.randn(B, T * G, H, D, generator=gen)).bfloat16().to(gpu_device)
    k = (0.5 * torch.randn(B, T, H, D, generator=gen)).bfloat16().to(gpu_device)
    v = (0.5 * torch.randn(B, T, H, D, generator=gen)).bfloat16().to(gpu_device)
    layers = [((0.5 * torch.randn(B, T, H, D, generator=gen)).bfloat16().to(gpu_device),
               (0.5 * torch.randn(B, T, H, D, generator=gen)).bfloat16().to(gpu_device)) for _ in range(Lmax)]
    cache = moda_amd.DepthCache(B, T, Lmax, H, D, torch.bfloat16, gpu_device)
    for n in range(1, Lmax + 1):
        cache.append(*layers[n - 1])
        ck, cv, nv = cache.filled()
        assert nv == n
        with torch.no_grad():
            o_inplace = moda_amd.parallel_moda(q, k, v, cached_k=ck, cached_v=cv, moda_group_num=G, depth_valid=nv)
            rk, rv = moda_amd.build_depth_cache(layers[:n])
            o_rebuilt = moda_amd.parallel_moda(q, k, v, cached_k=rk, cached_v=rv, moda_group_num=G)
        assert (o_inplace.float() - o_rebuilt.float()).abs().max().item() <= 2.0 ** -6, n


@pytest.mark.parametrize("case", [
    # (B, T, H, D, L, G, mode, dtype)
    (2, 150, 2, 64, 5, 2, "causal", torch.bfloat16),
    (1, 197, 1, 64, 12, 4, "noncausal", torch.float16),
    (1, 130, 2, 128, 4, 4, "causal", torch.bfloat16),
    (2, 60, 2, 128, 3, 1, "depth_only", torch.bfloat16),
    (1, 50, 2, 96, 3, 2, "causal", torch.bfloat16),     # matrix kernels, head dim zero-padded to 128
    (1, 50, 2, 36, 3, 2, "causal", torch.bfloat16),     # vector-ALU kernels (head dim not a multiple of 8)
    (2, 40, 1, 32, 4, 2, "noncausal", torch.float32),   # vector-ALU kernels (fp32)
    # chunk-visible: the chunk kernel, depth column tiles (narrow and 256-wide tiles), vector-ALU kernels
    (1, 150, 2, 128, 4, 4, "chunk_visible:16", torch.bfloat16),
    (1, 200, 1, 64, 3, 4, "chunk_visible:40", torch.float16),
    (1, 130, 2, 160, 3, 2, "chunk_visible:16", torch.bfloat16),
    (1, 60, 1, 32, 3, 2, "chunk_visible:8", torch.float32),
])
def test_depth_gradients_accumulate_over_layers(gpu_device, case):
    """The accumulate flag of the backward: the attention that saw n slots ADDS its depth gradients to slots
    < n of one shared buffer and leaves the other slots alone.  Layers L, L-1, ..., 1 (each with its own
    q, k, v, dO and depth_valid = n over one shared cache) run their backward in that order, as autograd
    would; the buffer must end up as the sum of the oracle's per-layer depth gradients (each evaluated on
    the compacted cache and scattered to its slots)."""
    from moda_amd import ops

    B, T, H, D, L, G, mode, dtype = case
    say(f"CASE accumulate-depth-grads {case}")
    cb = 0
    if ":" in mode:
        mode, cb = mode.split(":")[0], int(mode.split(":")[1])
    m = MODE_ID[mode]
    scale = D ** -0.5
    base = oracle.make_inputs(B, T, H, D, L, G, seed=61, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    kd, vd = base["kd"], base["vd"]
    acc_k = torch.zeros_like(kd).to(gpu_device)
    acc_v = torch.zeros_like(vd).to(gpu_device)
    ref_k = torch.zeros(kd.shape, dtype=torch.float32)
    ref_v = torch.zeros(vd.shape, dtype=torch.float32)
    kd_dev, vd_dev = kd.to(gpu_device), vd.to(gpu_device)
    for n in range(L, 0, -1):
        layer = oracle.make_inputs(B, T, H, D, L, G, seed=100 + n, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
        comp = dict(layer)
        comp["kd"] = oracle.compact_depth(kd, T, n).contiguous()
        comp["vd"] = oracle.compact_depth(vd, T, n).contiguous()
        ref = oracle.moda_dense_fwd_bwd(comp, scale, G, mode, cb)
        ref_k += oracle.scatter_depth_grad(ref["dkd"], T, L).float()
        ref_v += oracle.scatter_depth_grad(ref["dvd"], T, L).float()
        dev = to_dev(layer, gpu_device)
        o, lse = ops._raw_fwd(m, dev["q"], dev["k"], dev["v"], kd_dev, vd_dev, scale, G, cb, depth_valid=n)
        dq = torch.empty_like(dev["q"])
        dk = None if dev["k"] is None else torch.empty_like(dev["k"])
        dv = None if dev["v"] is None else torch.empty_like(dev["v"])
        ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], kd_dev, vd_dev, o, lse, dev["do"], scale, G, cb,
                     out=(dq, dk, dv, acc_k, acc_v), depth_valid=n, accumulate_depth=True)
        check("dq", dq, ref["dq"], dtype, f"layer {n}")
    # L additions, each rounded to the tensor type: the tolerance of one rounding per addition
    atol, rtol = TOL[dtype]
    for name, got, want in (("dkd", acc_k, ref_k), ("dvd", acc_v, ref_v)):
        err = (got.float().cpu() - want).abs()
        bound = atol + L * rtol * want.abs()
        assert bool((err <= bound).all()), f"{name}: max |err| {err.max():.3e}"
        rel = (got.float().cpu() - want).norm() / want.norm()
        assert rel <= 1e-2, (name, float(rel))


@pytest.mark.parametrize("case", [
    # (B, T, H, D, L, G, mode, dtype)
    (1, 1024, 1, 64, 2, 4, "causal", torch.bfloat16),      # 8 key tiles, four row segments each
    (1, 1100, 2, 128, 0, 2, "causal", torch.float16),      # ragged last tile, two segments
    (1, 1024, 2, 128, 1, 2, "noncausal", torch.bfloat16),
    (1, 1024, 1, 128, 3, 4, "chunk_visible", torch.bfloat16),
    (1, 1024, 1, 96, 1, 4, "causal", torch.bfloat16),      # padded head dim: the partial sums use the tile width
])
def test_row_split_sequence_gradients(gpu_device, case):
    """Launches with few key tiles cut every tile's query rows into segments that leave fp32 partial sums for a
    second kernel to add (shapes chosen so that the split is taken).  Checked against the oracle like every other
    case, and against the unsplit evaluation the same library gives with a workspace that only holds the row sums."""
    import ctypes

    from moda_amd import _lib, ops

    B, T, H, D, L, G, mode, dtype = case
    say(f"CASE row-split {case}")
    cb = 16 if mode == "chunk_visible" else 0
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=83, dtype=dtype, std=0.5)
    sc = D ** -0.5
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, mode, cb)
    dev = to_dev(inp, gpu_device)
    m = MODE_ID[mode]
    ws = ops.bwd_workspace(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], G, cb)
    rows_only = B * H * T * G * 4
    assert ws.numel() > rows_only + 256, "this shape was meant to take the row split"
    got = run_hip(dev, sc, G, mode, cb)
    compare_all(got, ref, dtype, f"row-split {case}")
    small = torch.empty(rows_only, dtype=torch.uint8, device=gpu_device)
    dq, dk, dv, dkd, dvd = ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], got["o"], got["lse"],
                                        dev["do"], sc, G, cb, ws=small)
    assert torch.equal(dq, got["dq"])
    check("dk", dk, ref["dk"], dtype, "unsplit")
    check("dv", dv, ref["dv"], dtype, "unsplit")
    # the two evaluations agree to a rounding or two of the 16-bit result (the unsplit launch of a short 64-wide case
    # runs on the short-launch kernel, which rounds P once where the split kernel rounds it twice)
    for a, b_ in ((dk, got["dk"]), (dv, got["dv"])):
        assert ((a.float() - b_.float()).abs() <= 2.0 ** -6 * b_.float().abs() + 2e-3).all()


def test_hip_graph_capture_and_replay(gpu_device):
    """Forward + backward captured in a HIP graph (the library allocates nothing and clears nothing, so
    every launch is capturable) and replayed with new inputs; every replay is checked against eager."""
    import moda_amd

    B, T, H, D, L, G = 1, 384, 2, 128, 4, 2
    scale = D ** -0.5
    gen = torch.Generator().manual_seed(37)

    def draw():
        i = oracle.make_inputs(B, T, H, D, L, G, seed=int(torch.randint(1 << 30, (1,), generator=gen)),
                               dtype=torch.bfloat16, std=0.5)
        return to_dev(i, gpu_device)

    static = draw()

    def step(x):
        o, lse = moda_amd.parallel_moda_fwd(x["q"], x["k"], x["v"], None, scale, cached_k=x["kd"], cached_v=x["vd"],
                                            moda_group_num=G)
        grads = moda_amd.parallel_moda_bwd(x["q"], x["k"], x["v"], o, None, lse, x["do"], scale, cached_k=x["kd"],
                                           cached_v=x["vd"], moda_group_num=G)
        return (o, lse) + tuple(g for g in grads if g is not None)

    side = torch.cuda.Stream(device=gpu_device)
    side.wait_stream(torch.cuda.current_stream(gpu_device))
    with torch.cuda.stream(side):
        for _ in range(2):
            step(static)  # warm-up outside capture: one-time kernel attribute setup
    torch.cuda.current_stream(gpu_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(static)
    for rep in range(3):
        fresh = draw()
        for n in static:
            static[n].copy_(fresh[n])
        graph.replay()
        torch.cuda.synchronize()
        eager = step(fresh)
        torch.cuda.synchronize()
        for a, b in zip(captured, eager):
            assert torch.equal(a, b), rep


# ---------------------------------------------------------------------------
# value head dim different from the key head dim (o [B, T*G, H, V], moda_v14.py:2792-2815)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("case", [
    (2, 70, 2, 64, 128, 3, 2, "causal", 0, torch.bfloat16),
    (1, 130, 1, 128, 64, 5, 4, "noncausal", 0, torch.float16),
    (1, 50, 2, 32, 96, 2, 1, "chunk_visible", 8, torch.float32),
    (1, 40, 2, 64, 32, 4, 2, "depth_only", 0, torch.bfloat16),
    (1, 33, 1, 96, 256, 0, 2, "causal", 0, torch.bfloat16),
    (2, 300, 2, 128, 64, 6, 4, "chunk_visible", 16, torch.bfloat16),   # chunk kernel
    (1, 260, 1, 40, 64, 3, 4, "chunk_visible", 40, torch.float16),     # depth column tiles, ring depth tiles
    (1, 1024, 1, 128, 32, 2, 4, "causal", 0, torch.bfloat16),          # row segments + reduce
    (3, 2100, 1, 64, 128, 2, 2, "causal", 0, torch.bfloat16),          # the throughput launch shape
    (1, 200, 2, 72, 36, 3, 2, "causal", 0, torch.bfloat16),            # value head dim not a multiple of 8: vector-ALU kernels
], ids=lambda c: f"{c[7]}-D{c[3]}-Dv{c[4]}")
def test_value_head_dim_differs_from_key_head_dim(gpu_device, case):
    import moda_amd

    B, T, H, D, Dv, L, G, mode, cb, dtype = case
    say(f"[Dv] {case}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=43, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"), Dv=Dv)
    sc = D ** -0.5
    ref = oracle.moda_dense_fwd_bwd(inp, sc, G, mode, cb)
    got = run_hip(to_dev(inp, gpu_device), sc, G, mode, cb)
    assert got["o"].shape[-1] == Dv and got["dq"].shape[-1] == D
    compare_all(got, ref, dtype, str(case))
    if mode == "causal":  # and through the public interface
        dev = to_dev(inp, gpu_device)
        o = moda_amd.parallel_moda(dev["q"], dev["k"], dev["v"], cached_k=dev["kd"], cached_v=dev["vd"], moda_group_num=G)
        check("o", o, ref["o"], dtype, "public " + str(case))


# ---------------------------------------------------------------------------
# packed variable-length batches (cu_seqlens): the oracle evaluates every sequence on its own
# ---------------------------------------------------------------------------
PACKED = [
    # lengths (base tokens), H, D, L, G, mode, chunk_tokens, dtype
    ((300, 1, 0, 129, 64, 700), 2, 128, 3, 4, "causal", 0, torch.bfloat16),
    ((197, 197, 50), 3, 64, 12, 1, "noncausal", 0, torch.bfloat16),
    ((5, 260, 33), 2, 64, 2, 2, "noncausal", 0, torch.float16),
    ((130, 17, 400), 1, 128, 6, 4, "chunk_visible", 16, torch.bfloat16),
    ((64, 0, 65, 3), 2, 64, 5, 2, "chunk_visible", 32, torch.float16),
    ((100, 7, 260), 2, 128, 7, 2, "depth_only", 0, torch.bfloat16),
    ((1100,), 1, 128, 2, 1, "causal", 0, torch.bfloat16),
    ((3, 2, 1, 1, 40), 2, 64, 0, 2, "causal", 0, torch.bfloat16),
    ((70, 9, 31), 2, 32, 3, 2, "causal", 0, torch.float32),
    ((40, 55), 1, 96, 2, 1, "noncausal", 0, torch.bfloat16),
    # chunks below and above one query tile (the waves' own depth phase and the chunk kernel; depth tiles streamed
    # by the workgroup and depth column tiles in the dK/dV kernel)
    ((70, 200, 33), 1, 128, 5, 4, "chunk_visible", 8, torch.float16),
    ((130, 17, 400), 2, 64, 3, 4, "chunk_visible", 32, torch.bfloat16),
    # head dims above 128: with the host copy of the offsets that the Python wrapper always passes, one launch per
    # sequence on the fixed-length 256-wide matrix kernels (the packed instantiations of those kernels are
    # switched off); test_packed_wide_without_host_offsets covers the vector-ALU route of the bare C ABI
    ((130, 1, 0, 300, 65), 2, 256, 3, 2, "causal", 0, torch.bfloat16),
    ((70, 200, 33), 1, 192, 5, 4, "chunk_visible", 8, torch.float16),
    ((100, 7, 260), 2, 160, 4, 1, "depth_only", 0, torch.bfloat16),
]


# This packed case once ended in a GPU memory fault on the packed instantiations of the 256-wide matrix kernels
# (which are switched off since).  It is kept off every matrix-kernel route: it runs with device offsets only,
# i.e. on the vector-ALU kernels.
PACKED_VECTOR_ROUTE_ONLY = [((70, 200, 33), 1, 192, 5, 4, "chunk_visible", 8, torch.float16)]


def _cu(lengths):
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + n)
    return cu


@pytest.mark.parametrize("case", PACKED, ids=lambda c: f"{c[5]}-{'_'.join(map(str, c[0]))}-D{c[2]}-L{c[3]}-G{c[4]}")
def test_packed_variable_length_batches(gpu_device, case):
    from moda_amd import ops

    lengths, H, D, L, G, mode, cb, dtype = case
    say(f"[packed] {case}")
    cu = _cu(lengths)
    total = cu[-1]
    inp = oracle.make_inputs(1, total, H, D, L, G, seed=29, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    ref = oracle.moda_packed_fwd_bwd(inp, cu, sc, G, mode, cb)
    dev = to_dev(inp, gpu_device)
    packed = ops._packed(torch.tensor(cu, device=gpu_device), dev["q"], G)
    assert (packed.n, packed.max_len, packed.total) == (len(lengths), max(lengths), total)
    if case in PACKED_VECTOR_ROUTE_ONLY:
        packed = packed._replace(host=None)
    m = MODE_ID[mode]
    o, lse = ops._raw_fwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], sc, G, cb, packed=packed)
    dq, dk, dv, dkd, dvd = ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], o, lse, dev["do"], sc, G,
                                        cb, packed=packed)
    got = {"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}
    compare_all(got, ref, dtype, str(case))


def test_packed_wide_without_host_offsets(gpu_device):
    """A packed batch with a head dim above 128 whose descriptor carries the device offsets only runs on the
    vector-ALU kernels; with the host copy it runs per sequence on the matrix kernels.  Both match the oracle."""
    from moda_amd import ops

    lengths, H, D, L, G, mode, cb, dtype = (40, 0, 75), 2, 160, 3, 2, "causal", 0, torch.bfloat16
    cu = _cu(lengths)
    inp = oracle.make_inputs(1, cu[-1], H, D, L, G, seed=31, dtype=dtype, std=0.5)
    sc = D ** -0.5
    ref = oracle.moda_packed_fwd_bwd(inp, cu, sc, G, mode, cb)
    dev = to_dev(inp, gpu_device)
    full = ops._packed(torch.tensor(cu, device=gpu_device), dev["q"], G)
    assert full.host is not None and ops._matrix_core_path(dev["q"], dev["v"], full)
    bare = full._replace(host=None)
    assert not ops._matrix_core_path(dev["q"], dev["v"], bare)
    for name, packed in (("per-sequence", full), ("device-offsets-only", bare)):
        say(f"[packed wide] {name}")
        o, lse = ops._raw_fwd(MODE_ID[mode], dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], sc, G, cb, packed=packed)
        dq, dk, dv, dkd, dvd = ops._raw_bwd(MODE_ID[mode], dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], o, lse,
                                            dev["do"], sc, G, cb, packed=packed)
        compare_all({"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}, ref, dtype, name)


def _random_packed_case(seed):
    import random

    rnd = random.Random(seed)
    mode = rnd.choice(["causal", "noncausal", "chunk_visible", "chunk_visible", "depth_only"])
    D = rnd.choice([32, 64, 64, 96, 128, 128, 160, 256])
    G = rnd.choice([1, 2, 4, 8])
    H = rnd.choice([1, 2])
    L = rnd.choice([0, 2, 5]) if mode != "depth_only" else rnd.choice([2, 5])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    n = rnd.randint(1, 5)
    cap = 1600 // G  # keeps every sequence's dense oracle small
    lengths = tuple(rnd.choice([0, 1, 17, 64, 65, 130, 200, 333, 400][: 9 if cap >= 400 else 7]) for _ in range(n))
    if sum(lengths) == 0:
        lengths = lengths + (33,)
    cb = rnd.choice([1, 8, 16, max(1, 64 // G), max(1, 128 // G), 40]) if mode == "chunk_visible" else 0
    return lengths, H, D, L, G, mode, cb, dtype


@pytest.mark.parametrize("seed", range(24))
def test_random_sweep_packed(gpu_device, seed):
    """Random packed batches on the 64- and 128-wide tiles: empty and one-token sequences, chunks below and above
    one query tile, every mode."""
    test_packed_variable_length_batches(gpu_device, _random_packed_case(7000 + seed))


def test_packed_batch_equals_separate_calls_bitwise(gpu_device):
    """One launch over the packed batch returns, bit for bit, what one call per sequence returns; also
    through the public autograd interface with an int64 cu_seqlens as callers of fla pass it."""
    import moda_amd

    lengths, H, D, L, G = (333, 64, 1, 520), 2, 128, 4, 4
    cu = _cu(lengths)
    inp = to_dev(oracle.make_inputs(1, cu[-1], H, D, L, G, seed=31, dtype=torch.bfloat16, std=0.5), gpu_device)
    leaf = {n: inp[n].clone().requires_grad_(True) for n in ("q", "k", "v", "kd", "vd")}
    o, lse = moda_amd.parallel_moda(leaf["q"], leaf["k"], leaf["v"], cached_k=leaf["kd"], cached_v=leaf["vd"],
                                    moda_group_num=G, need_lse=True,
                                    cu_seqlens=torch.tensor(cu, dtype=torch.int64, device=gpu_device))
    (o * inp["do"]).sum().backward()
    mult = {"q": G, "k": 1, "v": 1, "kd": L, "vd": L}
    for i in range(len(lengths)):
        a, b = cu[i], cu[i + 1]
        part = {n: inp[n][:, a * m:b * m] for n, m in mult.items()}
        part["do"] = inp["do"][:, a * G:b * G]
        # (the packed launch sums dk, dv in one pass per key tile: ask the separate calls for the same order)
        one = run_hip(part, D ** -0.5, G, "causal", no_row_split=True)
        assert torch.equal(o[:, a * G:b * G], one["o"]) and torch.equal(lse[:, a * G:b * G], one["lse"]), i
        for n, key in (("q", "dq"), ("k", "dk"), ("v", "dv"), ("kd", "dkd"), ("vd", "dvd")):
            assert torch.equal(leaf[n].grad[:, a * mult[n]:b * mult[n]], one[key]), (i, n)


def test_packed_batch_on_the_narrow_tiles_against_separate_calls(gpu_device):
    """On the 64-wide tiles the separate (short) calls form dk, dv in the four-wave kernel, which rounds the
    probabilities once; this packed launch (longest sequence above 512 query rows, few column tiles) in the
    role-split kernel, which rounds them twice: everything else is bit-identical, dk and dv agree to that rounding."""
    lengths, H, D, L, G = (197, 64, 1, 300), 2, 64, 4, 2
    cu = _cu(lengths)
    inp = to_dev(oracle.make_inputs(1, cu[-1], H, D, L, G, seed=41, dtype=torch.bfloat16, std=0.5), gpu_device)
    from moda_amd import ops

    m = MODE_ID["causal"]
    packed = ops._packed(torch.tensor(cu, device=gpu_device), inp["q"], G)
    o, lse = ops._raw_fwd(m, inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], D ** -0.5, G, 0, packed=packed)
    grads = ops._raw_bwd(m, inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], o, lse, inp["do"], D ** -0.5, G, 0,
                         packed=packed)
    whole = dict(zip(("o", "lse", "dq", "dk", "dv", "dkd", "dvd"), (o, lse) + tuple(grads)))
    mult = {"q": G, "k": 1, "v": 1, "kd": L, "vd": L}
    for i in range(len(lengths)):
        a, b = cu[i], cu[i + 1]
        part = {n: inp[n][:, a * m:b * m] for n, m in mult.items()}
        part["do"] = inp["do"][:, a * G:b * G]
        one = run_hip(part, D ** -0.5, G, "causal", no_row_split=True)
        for key, m in (("o", G), ("lse", G), ("dq", G), ("dkd", L), ("dvd", L)):
            assert torch.equal(whole[key][:, a * m:b * m], one[key]), (i, key)
        for key in ("dk", "dv"):
            got, want = whole[key][:, a:b].float(), one[key].float()
            assert ((got - want).abs() <= 2.0 ** -6 * want.abs() + 2e-3).all(), (i, key)


def test_packed_plain_gqa_attention(gpu_device):
    import moda_amd

    lengths, Hkv, G, D = (200, 77, 300), 2, 4, 128
    cu = _cu(lengths)
    inp = oracle.make_inputs(1, cu[-1], Hkv, D, 0, G, seed=37, dtype=torch.bfloat16, std=0.5, Hq=Hkv * G)
    dev = to_dev(inp, gpu_device)
    dl = {n: dev[n].clone().requires_grad_(True) for n in ("q", "k", "v")}
    o = moda_amd.parallel_attn(dl["q"], dl["k"], dl["v"], cu_seqlens=torch.tensor(cu, device=gpu_device))
    (o * dev["do"]).sum().backward()
    for i in range(len(lengths)):
        a, b = cu[i], cu[i + 1]
        leaf = {n: inp[n][:, a:b].float().clone().requires_grad_(True) for n in ("q", "k", "v")}
        o_ref, _ = oracle.plain_gqa_dense(leaf["q"], leaf["k"], leaf["v"])
        (o_ref * inp["do"][:, a:b].float()).sum().backward()
        check("o", o[:, a:b], o_ref, torch.bfloat16, f"packed plain {i}")
        for n in ("q", "k", "v"):
            check("d" + n, dl[n].grad[:, a:b], leaf[n].grad, torch.bfloat16, f"packed plain {i}")


# ---------------------------------------------------------------------------
# the attention module and the depth-stream manager around the operator
# ---------------------------------------------------------------------------
def _oracle_parallel_moda(q, k, v, g=None, scale=None, cu_seqlens=None, cached_k=None, cached_v=None, moda_group_num=1,
                          is_causal=True, head_first=False, warn_shape=True, depth_valid=None):
    """What the module calls, answered by the oracle's dense form in fp32 and rounded to the input type."""
    assert depth_valid is None
    o, _ = oracle.moda_dense(q, k, v, cached_k, cached_v, scale, moda_group_num, "causal" if is_causal else "noncausal")
    return o.to(q.dtype)


def _oracle_parallel_moda_chunk_visible(q, k, v, g=None, scale=None, cu_seqlens=None, cached_k=None, cached_v=None,
                                        moda_group_num=1, head_first=False, warn_shape=True, chunk_rows=None,
                                        depth_valid=None):
    assert depth_valid is None
    o, _ = oracle.moda_dense(q, k, v, cached_k, cached_v, scale, moda_group_num, "chunk_visible",
                             (chunk_rows or 64) // moda_group_num)
    return o.to(q.dtype)


@pytest.mark.parametrize("variant", [
    # (causal, post_norm, ffn_kv, chunk rows or None)
    (False, False, False, None), (True, False, False, None), (False, True, False, None), (True, False, True, None),
    (False, True, True, None), (True, False, False, 32), (True, True, True, 64),
], ids=lambda v: f"{'causal' if v[0] else 'noncausal'}{'-postnorm' if v[1] else ''}{'-ffnkv' if v[2] else ''}"
                 f"{'-chunk%d' % v[3] if v[3] else ''}")
def test_attention_stack_with_depth_stream(gpu_device, monkeypatch, variant):
    """A three-block stack (layer norm, MoDAAttention, MLP, one DepthStream; pre- or post-norm, optionally
    with K/V of the block output pushed as well) trained one step on the HIP operator with the in-place depth
    stream (one cache, one gradient buffer, no per-layer rebuild), against the same torch modules with the
    oracle answering every attention call and torch.stack building the cache; also the rebuilding path and
    the no-grad path (in-place cache, depth_valid)."""
    import moda_amd
    from moda_amd import depth_cache, modules

    causal, post_norm, ffn_kv, chunk_rows = variant
    torch.manual_seed(41)
    dim, depth, heads, kv_heads, B, N = 256, 3, 4, 2, 2, 70
    model = moda_amd.MoDAStack(dim, depth, heads, kv_heads, is_causal=causal, post_norm=post_norm,
                               ffn_kv=ffn_kv, chunk_rows=chunk_rows).to(gpu_device).to(torch.bfloat16)
    x = (0.5 * torch.randn(B, N, dim, device=gpu_device)).to(torch.bfloat16)
    w = torch.randn(B, N, dim, device=gpu_device).to(torch.bfloat16)

    def step(inplace=None):
        model.zero_grad(set_to_none=True)
        xin = x.clone().requires_grad_(True)
        y = model(xin, inplace_cache=inplace)
        (y.float() * w.float()).sum().backward()
        grads = {n: (p.grad if p.grad is not None else torch.zeros_like(p)).float().clone()
                 for n, p in model.named_parameters()}
        return y.detach().float(), xin.grad.float(), grads

    # the in-place training path must not rebuild the cache: count stack_depth calls
    calls = {"n": 0}
    real_stack = modules.stack_depth

    def counting_stack(layers):
        calls["n"] += 1
        return real_stack(layers)

    monkeypatch.setattr(modules, "stack_depth", counting_stack)
    y_hip, dx_hip, g_hip = step()
    assert calls["n"] == 0, "the in-place depth stream rebuilt the cache"
    y_rb, dx_rb, g_rb = step(inplace=False)
    assert calls["n"] > 0
    with torch.no_grad():
        y_inplace = model(x).float()
    monkeypatch.setattr(modules, "parallel_moda", _oracle_parallel_moda)
    monkeypatch.setattr(modules, "parallel_moda_chunk_visible", _oracle_parallel_moda_chunk_visible)
    monkeypatch.setattr(modules, "stack_depth", lambda layers: oracle.depth_cache_ref(list(layers)))
    y_ref, dx_ref, g_ref = step(inplace=False)

    def close(a, b, what, tol=1.5e-2):
        rel = ((a - b).norm() / b.norm().clamp_min(1e-6)).item()
        assert rel <= tol, (what, rel)

    close(y_hip, y_ref, "y")
    close(y_rb, y_ref, "y (rebuilt cache)")
    close(y_inplace, y_ref, "y (in-place depth cache, no grad)")
    close(dx_hip, dx_ref, "dx")
    close(dx_rb, dx_ref, "dx (rebuilt cache)")
    for n in g_ref:
        close(g_hip[n], g_ref[n], n)
        close(g_rb[n], g_ref[n], n + " (rebuilt cache)")
    # every projection that feeds the depth stream received a gradient through it
    assert g_hip["blocks.0.attn.kv.weight"].abs().max() > 0
    if ffn_kv:
        assert g_hip["blocks.0.attn.kv_ffn.weight"].abs().max() > 0
        # the last block's FFN K/V are pushed after the last attention call: nothing reads them
        assert g_hip[f"blocks.{depth - 1}.attn.kv_ffn.weight"].abs().max() == 0


# ---------------------------------------------------------------------------
# the throughput launch shape (256-row workgroups, ping-pong halves) on short and ragged sequences: enough
# (batch, head) pairs that the small-problem shape is not chosen
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("case", [
    (64, 1, 8, 64, 2, 1, "causal", 0, torch.bfloat16),
    (64, 63, 8, 64, 0, 1, "causal", 0, torch.bfloat16),
    (64, 130, 8, 64, 3, 2, "causal", 0, torch.float16),
    (32, 300, 16, 128, 5, 4, "noncausal", 0, torch.bfloat16),
    (64, 129, 8, 128, 2, 2, "chunk_visible", 16, torch.bfloat16),
    (64, 65, 8, 128, 7, 4, "depth_only", 0, torch.float16),
    (128, 257, 4, 64, 1, 1, "causal", 0, torch.bfloat16),
    (32, 300, 16, 96, 3, 2, "causal", 0, torch.bfloat16),
    (64, 130, 8, 32, 2, 1, "noncausal", 0, torch.float16),
], ids=lambda c: f"{c[6]}-B{c[0]}-T{c[1]}-D{c[3]}-L{c[4]}-G{c[5]}")
def test_large_launch_shape_on_ragged_inputs(gpu_device, case):
    B, T, H, D, L, G, mode, cb, dtype = case
    say(f"[large shape] {case}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=53, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    dev = to_dev(inp, gpu_device)
    got = run_hip(dev, sc, G, mode, cb)
    ref = oracle.moda_dense_fwd_bwd(dev, sc, G, mode, cb)  # the oracle's dense form, evaluated on the device
    compare_all(got, ref, dtype, str(case))


# ---------------------------------------------------------------------------
# peaked softmax: logits of several dozen (base 2), where the lazily moved exponent reference, the
# 2^8 head room of the rounded probabilities and the fp16 range are all in play
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("case", [
    (1, 300, 2, 128, 4, 2, "causal", torch.bfloat16, 3.0),
    (1, 300, 2, 64, 4, 2, "causal", torch.float16, 3.0),
    (2, 200, 2, 128, 3, 4, "noncausal", torch.bfloat16, 4.0),
    (64, 130, 8, 64, 3, 2, "causal", torch.bfloat16, 3.0),
    (1, 257, 1, 128, 6, 1, "depth_only", torch.float16, 3.0),
    (1, 1000, 1, 128, 2, 1, "causal", torch.bfloat16, 6.0),
], ids=lambda c: f"{c[6]}-T{c[1]}-D{c[3]}-std{c[8]}-{str(c[7])[6:]}")
def test_peaked_softmax(gpu_device, case):
    B, T, H, D, L, G, mode, dtype, std = case
    say(f"[peaked] {case}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=5, dtype=dtype, std=std, depth_only=(mode == "depth_only"))
    for n in ("v", "vd"):  # values stay of order one: the test is about the softmax
        if inp[n] is not None:
            inp[n] = (inp[n].float() / std).to(dtype)
    dev = to_dev(inp, gpu_device)
    got = run_hip(dev, D ** -0.5, G, mode)
    ref = oracle.moda_dense_fwd_bwd(dev, D ** -0.5, G, mode)
    assert ref["lse"].abs().max() > 40  # the case is what it claims to be
    # Gradients here are sums of terms of order ten that cancel; P and dS are rounded to the 16-bit input
    # type before the second product (as in the reference, moda_v14.py:209, 712), so the error of an
    # element scales with the tensor's magnitude, not with the element's: bound it by atol + rtol * max|ref|.
    atol, rtol = TOL[dtype]
    for n in ("o", "dq", "dk", "dv", "dkd", "dvd"):
        if ref[n] is None:
            continue
        g, r = got[n].float(), ref[n].float()
        assert torch.isfinite(g).all(), n
        bound = atol + rtol * r.abs().max().item()
        assert (g - r).abs().max().item() <= bound, (n, (g - r).abs().max().item(), bound)
    check("lse", got["lse"], ref["lse"], dtype, str(case))


# ---------------------------------------------------------------------------
# seeded random sweep over shapes, modes and options (ragged sizes, every option combined)
# ---------------------------------------------------------------------------
def _random_case(seed):
    import random

    rnd = random.Random(seed)
    mode = rnd.choice(["causal", "causal", "noncausal", "chunk_visible", "depth_only"])
    D = rnd.choice([64, 128])
    G = rnd.choice([1, 2, 4, 8])
    H = rnd.choice([1, 2, 3])
    L = rnd.choice([0, 1, 2, 3, 5, 9]) if mode != "depth_only" else rnd.choice([1, 2, 5, 9])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    packed = rnd.random() < 0.4
    if packed:
        lengths = [rnd.choice([0, 1, 2, 17, 63, 64, 65, 130, 257]) for _ in range(rnd.randint(1, 4))]
        if sum(lengths) == 0:
            lengths[0] = 33
        B = 1
    else:
        lengths = [rnd.choice([1, 2, 3, 31, 64, 65, 127, 129, 200, 301])]
        B = rnd.choice([1, 2])
    cb = rnd.choice([1, 2, 16, 64 // G if 64 // G > 0 else 1]) if mode == "chunk_visible" else 0
    valid = None
    if L > 1 and mode != "chunk_visible" and rnd.random() < 0.4:
        valid = rnd.randint(1, L)
    return mode, D, G, H, L, dtype, packed, lengths, B, cb, valid


@pytest.mark.parametrize("seed", range(48))
def test_random_sweep(gpu_device, seed):
    from moda_amd import ops

    mode, D, G, H, L, dtype, packed, lengths, B, cb, valid = _random_case(1000 + seed)
    say(f"[sweep {seed}] mode={mode} D={D} G={G} H={H} L={L} {dtype} packed={packed} lengths={lengths} B={B} cb={cb} valid={valid}")
    total = sum(lengths)
    inp = oracle.make_inputs(B, total, H, D, L, G, seed=seed, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    ref_inp = dict(inp)
    if valid is not None:
        ref_inp["kd"] = oracle.compact_depth(inp["kd"], total, valid)
        ref_inp["vd"] = oracle.compact_depth(inp["vd"], total, valid)
    cu = _cu(lengths)
    if packed:
        ref = oracle.moda_packed_fwd_bwd(ref_inp, cu, sc, G, mode, cb)
    else:
        ref = oracle.moda_dense_fwd_bwd(ref_inp, sc, G, mode, cb)
    if valid is not None:
        ref["dkd"] = oracle.scatter_depth_grad(ref["dkd"], total, L)
        ref["dvd"] = oracle.scatter_depth_grad(ref["dvd"], total, L)
    dev = to_dev(inp, gpu_device)
    pk = ops._packed(torch.tensor(cu, device=gpu_device), dev["q"], G) if packed else None
    m = MODE_ID[mode]
    o, lse = ops._raw_fwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], sc, G, cb, depth_valid=valid, packed=pk)
    dq, dk, dv, dkd, dvd = ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], o, lse, dev["do"], sc, G,
                                        cb, depth_valid=valid, packed=pk)
    got = {"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}
    compare_all(got, ref, dtype, f"sweep {seed}")


def _random_case_wide(seed, dims=(8, 32, 64, 72, 96, 128)):
    """A second family: head dims below the tile widths, sequences long enough for the row split of the dK/dV
    kernel, chunks above and below one query tile."""
    import random

    rnd = random.Random(seed)
    mode = rnd.choice(["causal", "noncausal", "chunk_visible", "chunk_visible", "depth_only"])
    D = rnd.choice(list(dims))
    G = rnd.choice([1, 2, 4, 8, 16])
    H = rnd.choice([1, 2])
    L = rnd.choice([0, 1, 3, 6]) if mode != "depth_only" else rnd.choice([1, 3, 6])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    T = rnd.choice([40, 129, 300, 520, 700, 1100])
    if mode == "depth_only":
        T = min(T, 520)
    T = min(T, 4400 // G)  # keeps the dense oracle's score matrix small
    B = rnd.choice([1, 2]) if T * G <= 2400 else 1
    cb = rnd.choice([1, 4, 16, max(1, 64 // G), max(1, 128 // G), 40]) if mode == "chunk_visible" else 0
    valid = None
    if L > 1 and mode != "chunk_visible" and rnd.random() < 0.3:
        valid = rnd.randint(1, L)
    return mode, D, G, H, L, dtype, T, B, cb, valid


@pytest.mark.parametrize("seed", range(64))
def test_random_sweep_wide(gpu_device, seed):
    """Seeds 40 and up draw head dims above 128 (the 256-wide tiles: 16 query rows per wave, 64-column workgroups
    and 32-row query tiles in the dK/dV kernel)."""
    from moda_amd import ops

    dims = (8, 32, 64, 72, 96, 128) if seed < 40 else (136, 160, 192, 200, 256, 256)
    mode, D, G, H, L, dtype, T, B, cb, valid = _random_case_wide(5000 + seed, dims)
    say(f"[wide sweep {seed}] mode={mode} D={D} G={G} H={H} L={L} {dtype} T={T} B={B} cb={cb} valid={valid}")
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=seed, dtype=dtype, std=0.5, depth_only=(mode == "depth_only"))
    sc = D ** -0.5
    ref_inp = dict(inp)
    if valid is not None:
        ref_inp["kd"] = oracle.compact_depth(inp["kd"], T, valid)
        ref_inp["vd"] = oracle.compact_depth(inp["vd"], T, valid)
    ref = oracle.moda_dense_fwd_bwd(ref_inp, sc, G, mode, cb)
    if valid is not None:
        ref["dkd"] = oracle.scatter_depth_grad(ref["dkd"], T, L)
        ref["dvd"] = oracle.scatter_depth_grad(ref["dvd"], T, L)
    dev = to_dev(inp, gpu_device)
    m = MODE_ID[mode]
    o, lse = ops._raw_fwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], sc, G, cb, depth_valid=valid)
    dq, dk, dv, dkd, dvd = ops._raw_bwd(m, dev["q"], dev["k"], dev["v"], dev["kd"], dev["vd"], o, lse, dev["do"], sc, G,
                                        cb, depth_valid=valid)
    got = {"o": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv, "dkd": dkd, "dvd": dvd}
    compare_all(got, ref, dtype, f"wide sweep {seed}")


def test_more_than_65535_batch_heads(gpu_device):
    """Launch grids are one-dimensional: batch x heads beyond the 65535 limit of a grid's y extent."""
    B, T, H, D, L, G = 70000, 3, 1, 64, 2, 2
    inp = oracle.make_inputs(B, T, H, D, L, G, seed=47, dtype=torch.bfloat16, std=0.5)
    ref = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, "causal")
    got = run_hip(to_dev(inp, gpu_device), D ** -0.5, G, "causal")
    compare_all(got, ref, torch.bfloat16, "many batch-heads")


def test_empty_and_degenerate(gpu_device):
    import moda_amd

    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=gpu_device)
    o = moda_amd.parallel_moda(z(0, 8, 2, 64), z(0, 8, 2, 64), z(0, 8, 2, 64))
    assert o.shape == (0, 8, 2, 64)
    o = moda_amd.parallel_moda(z(1, 0, 2, 64), z(1, 0, 2, 64), z(1, 0, 2, 64), warn_shape=False)
    assert o.shape == (1, 0, 2, 64)
    # constant values => constant output, exactly representable
    q = torch.randn(1, 40, 2, 64, device=gpu_device).bfloat16()
    k = torch.randn(1, 20, 2, 64, device=gpu_device).bfloat16()
    v = torch.full((1, 20, 2, 64), 1.5, device=gpu_device).bfloat16()
    kd = torch.randn(1, 60, 2, 64, device=gpu_device).bfloat16()
    vd = torch.full((1, 60, 2, 64), 1.5, device=gpu_device).bfloat16()
    o = moda_amd.parallel_moda(q, k, v, cached_k=kd, cached_v=vd, moda_group_num=2)
    assert (o.float() - 1.5).abs().max() <= 2.0 ** -6


# ---------------------------------------------------------------------------
# depth-KV reorganisation: bit-exact permutation
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(2, 197, 6, 64, 12, torch.bfloat16), (1, 1024, 4, 128, 24, torch.bfloat16),
                                   (3, 5, 1, 20, 3, torch.float16), (1, 7, 3, 6, 70, torch.float32),
                                   (2, 16, 2, 64, 1, torch.float32)])
def test_depth_reorg_bit_exact(gpu_device, shape):
    import moda_amd

    B, T, H, D, L, dtype = shape
    gen = torch.Generator().manual_seed(1)
    layers = [torch.randn(B, T, H, D, generator=gen).to(dtype) for _ in range(L)]
    dev_layers = [x.to(gpu_device).requires_grad_(True) for x in layers]
    cache = moda_amd.stack_depth(dev_layers)
    ref = oracle.depth_cache_ref(layers)
    assert torch.equal(cache.cpu(), ref)
    g = torch.randn(B, T * L, H, D, generator=gen).to(dtype)
    cache.backward(g.to(gpu_device))
    back = oracle.depth_cache_grad_ref(g, L)
    for l in range(L):
        assert torch.equal(dev_layers[l].grad.cpu(), back[l])
    # in-place append builds the same cache
    dc = moda_amd.DepthCache(B, T, L, H, D, dtype, gpu_device)
    for l in range(L):
        dc.append(dev_layers[l].detach(), dev_layers[l].detach())
    kfull, vfull = dc.full()
    assert torch.equal(kfull.cpu(), ref) and torch.equal(vfull.cpu(), ref)


def test_depth_reorg_round_trip_full_size(gpu_device):
    """c3-sized cache: reorg then inverse reorg is the identity; checksum is preserved."""
    import moda_amd
    from moda_amd import depth_cache

    B, T, H, D, L = 1, 16384, 4, 128, 24
    layers = [torch.randn(B, T, H, D, device=gpu_device).bfloat16() for _ in range(L)]
    cache = moda_amd.stack_depth(layers)
    back = depth_cache._reorg_bwd(cache, L, 0, L, (B, T, H, D))
    for a, b in zip(layers, back):
        assert torch.equal(a, b)
    assert torch.equal(cache.view(B, T, L, H, D)[:, :, 7], layers[7])
