"""Every global-memory access of the matrix-core kernels, replayed on the CPU.

``tests/address_walker.cpp`` is compiled for the host (hipcc, host pass only: no GPU needed) together with the
kernels' own index arithmetic (``moda_amd/csrc/geometry.h``, ``kargs.h``, ``tile.h``, ``tile16.h``, ``tuning.h``)
and walks every (workgroup, wave, lane, trip) of a forward + backward launch: register operand loads, every tile
descriptor with each lane's vector and scalar offset (the lanes that fetch past the tensors' head dim included),
the row-statistics loads, the LDS targets against the launch's dynamic LDS size, and all stores; every output
element must be written exactly once.

The first case is the packed batch that once ended in a GPU memory fault on the packed instantiations of the
256-wide kernels (switched off since).  The walk finds every access of it inside its tensor: the fault is not an
error of the kernels' index arithmetic.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MODES = {"causal": 0, "noncausal": 1, "chunk_visible": 2, "depth_only": 3, "plain": 4}


@pytest.fixture(scope="module")
def walker(tmp_path_factory):
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not found")
    out = str(tmp_path_factory.mktemp("walker") / "address_walker")
    # host pass only, under AddressSanitizer (the walker's own tables and the kernels' index code run checked)
    checked = ["-fsanitize=address", "-fno-gpu-sanitize", "-fno-omit-frame-pointer"]  # host code only
    subprocess.run(["hipcc", "-x", "hip", "--cuda-host-only", "-std=c++17", "-O1", "-g", *checked,
                    os.path.join(ROOT, "tests", "address_walker.cpp"), "-o", out], check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    return out


def tile_width(D):
    return 64 if D <= 64 else 128 if D <= 128 else 256


def run(walker, lengths, H, D, L, G, mode, cb=0, packed=True, B=1, Lv=0, split=1, env=None, Dv=None):
    n = len(lengths) if packed else B
    Dv = D if Dv is None else Dv
    args = [walker, tile_width(max(D, Dv)), D, Dv, H, G, L, Lv, MODES[mode], cb, split, int(packed), n] + list(lengths)
    e = dict(os.environ)
    e.update(env or {})
    r = subprocess.run([str(x) for x in args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=e,
                       timeout=600)
    return r.returncode, r.stdout.strip() + r.stderr.strip()


FAULTED = dict(lengths=(70, 200, 33), H=1, D=192, L=5, G=4, mode="chunk_visible", cb=8)

PACKED = [
    # the packed cases of the GPU parity tests (tests/test_parity_gpu.py: PACKED), 16-bit head dims that are a
    # multiple of 8: lengths, H, D, L, G, mode, chunk tokens
    ((300, 1, 0, 129, 64, 700), 2, 128, 3, 4, "causal", 0),
    ((197, 197, 50), 3, 64, 12, 1, "noncausal", 0),
    ((5, 260, 33), 2, 64, 2, 2, "noncausal", 0),
    ((130, 17, 400), 1, 128, 6, 4, "chunk_visible", 16),
    ((64, 0, 65, 3), 2, 64, 5, 2, "chunk_visible", 32),
    ((100, 7, 260), 2, 128, 7, 2, "depth_only", 0),
    ((1100,), 1, 128, 2, 1, "causal", 0),
    ((3, 2, 1, 1, 40), 2, 64, 0, 2, "causal", 0),
    ((40, 55), 1, 96, 2, 1, "noncausal", 0),
    ((70, 200, 33), 1, 128, 5, 4, "chunk_visible", 8),
    ((130, 17, 400), 2, 64, 3, 4, "chunk_visible", 32),
    # the packed instantiations of the 256-wide kernels (not launched by the library)
    ((130, 1, 0, 300, 65), 2, 256, 3, 2, "causal", 0),
    ((100, 7, 260), 2, 160, 4, 1, "depth_only", 0),
    ((70, 200, 33), 2, 136, 3, 8, "chunk_visible", 4),
    ((333, 1, 64), 1, 248, 2, 2, "noncausal", 0),
]

FIXED = [
    # B, T, H, D, L, G, mode, chunk tokens, Lv
    (2, 150, 2, 64, 5, 2, "causal", 0, 0),
    (1, 197, 3, 128, 4, 1, "noncausal", 0, 0),
    (1, 300, 2, 128, 6, 4, "chunk_visible", 16, 0),
    (1, 260, 1, 64, 3, 4, "chunk_visible", 40, 0),
    (2, 60, 2, 128, 3, 1, "depth_only", 0, 0),
    (1, 333, 2, 128, 0, 4, "plain", 0, 0),
    (1, 200, 2, 120, 3, 4, "causal", 0, 0),
    (1, 90, 1, 8, 2, 2, "causal", 0, 0),
    (2, 64, 2, 64, 4, 2, "causal", 0, 2),          # partially filled depth stream: tile loads through the slot mapping
    (1, 150, 2, 128, 7, 4, "noncausal", 0, 3),
    (2, 100, 1, 64, 5, 1, "depth_only", 0, 1),
    (1, 300, 2, 128, 6, 4, "chunk_visible", 16, 4),  # ... chunks within one query tile (chunk kernel)
    (1, 260, 1, 64, 3, 4, "chunk_visible", 40, 2),   # ... and above it (ring depth tiles, depth column tiles)
    (1, 200, 2, 192, 5, 2, "chunk_visible", 16, 3),  # ... on the 256-wide tiles
    (2, 130, 2, 256, 12, 1, "causal", 0, 5),
    (2, 130, 2, 192, 6, 4, "chunk_visible", 16, 0),
    (1, 700, 1, 256, 3, 2, "chunk_visible", 64, 0),
    (1, 197, 3, 160, 12, 1, "noncausal", 0, 0),
    (1, 100, 2, 256, 7, 4, "depth_only", 0, 0),
    (1, 1, 1, 256, 1, 1, "causal", 0, 0),
    (3, 2100, 1, 128, 2, 2, "causal", 0, 0),       # the throughput launch shape (256 rows per workgroup)
    # query groups that fill a wave's 32 rows, or do not divide them (a token's rows then straddle waves and tiles)
    (1, 77, 2, 128, 5, 8, "causal", 0, 0),
    (1, 40, 1, 64, 3, 32, "noncausal", 0, 2),
    (2, 90, 2, 128, 4, 3, "causal", 0, 0),
    (1, 50, 1, 64, 6, 5, "depth_only", 0, 4),
    (2, 1500, 1, 128, 3, 4, "causal", 0, 2),       # ... in the throughput launch shape, partially filled
    # 64-wide tiles, more than 512 query rows, three sequence column tiles per compute unit: the four-wave dK/dV kernel
    (12, 1024, 8, 64, 2, 2, "causal", 0, 0),
    # what the per-sequence route launches for the packed case above: one fixed-length problem per sequence
    (1, 70, 1, 192, 5, 4, "chunk_visible", 8, 0),
    (1, 200, 1, 192, 5, 4, "chunk_visible", 8, 0),
    (1, 33, 1, 192, 5, 4, "chunk_visible", 8, 0),
]


def test_the_packed_wide_case_that_faulted_stays_inside_its_tensors(walker):
    rc, out = run(walker, **FAULTED)
    assert rc == 0 and out.startswith("OK"), out
    # ... and the walk is not vacuous: the same launch over tensors that are one row short is reported, whichever
    # tensor it is (a read through a tile descriptor, a register load, a store)
    for name, cut in (("kd", 192 * 2), ("q", 192 * 2), ("dvd", 192 * 2), ("lse", 4), ("delta", 4), ("do", 16), ("o", 8)):
        rc, out = run(walker, env={"WALKER_SHRINK": f"{name}:{cut}"}, **FAULTED)
        assert rc == 1 and "VIOLATION" in out, (name, out)


@pytest.mark.parametrize("case", PACKED, ids=lambda c: f"{c[5]}-{'_'.join(map(str, c[0]))}-D{c[2]}")
def test_packed_batches(walker, case):
    lengths, H, D, L, G, mode, cb = case
    rc, out = run(walker, lengths, H, D, L, G, mode, cb)
    assert rc == 0 and out.startswith("OK"), out


@pytest.mark.parametrize("case", FIXED, ids=lambda c: f"{c[6]}-B{c[0]}T{c[1]}H{c[2]}D{c[3]}L{c[4]}G{c[5]}")
def test_fixed_length_batches(walker, case):
    B, T, H, D, L, G, mode, cb, Lv = case
    rc, out = run(walker, (T,), H, D, L, G, mode, cb, packed=False, B=B, Lv=Lv)
    assert rc == 0 and out.startswith("OK"), out


@pytest.mark.parametrize("case", [
    # B, T, H, D, Dv, L, G, mode, chunk tokens, Lv: value head dim different from the key head dim (one tile width)
    (2, 150, 2, 64, 32, 5, 2, "causal", 0, 0),
    (1, 197, 3, 64, 128, 4, 1, "noncausal", 0, 0),
    (1, 300, 2, 128, 96, 6, 4, "chunk_visible", 16, 0),
    (1, 260, 1, 40, 64, 3, 4, "chunk_visible", 40, 2),
    (2, 60, 2, 128, 256, 3, 1, "depth_only", 0, 0),
    (1, 333, 2, 192, 64, 0, 4, "plain", 0, 0),
    (1, 2100, 1, 128, 64, 2, 2, "causal", 0, 1),
], ids=lambda c: f"{c[7]}-D{c[3]}-Dv{c[4]}")
def test_value_head_dim_differs(walker, case):
    B, T, H, D, Dv, L, G, mode, cb, Lv = case
    rc, out = run(walker, (T,), H, D, L, G, mode, cb, packed=False, B=B, Lv=Lv, Dv=Dv)
    assert rc == 0 and out.startswith("OK"), out


def test_row_split_launch(walker):
    """Light launches cut every key tile's query rows into segments (one workgroup each): the tile loads of every
    segment stay inside q, do, lse and the row sums."""
    for split in (2, 4, 8):
        rc, out = run(walker, (4096,), 1, 128, 0, 2, "causal", packed=False, B=1, split=split)
        assert rc == 0 and out.startswith("OK"), out
