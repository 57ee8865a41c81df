"""Headline benchmark: parallel_moda forward+backward TFLOP/s on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c3|c2|c5|c5fda|c4packed|plain]
                    [--no-cpu-baseline] [--no-configs] [--with-stack]
    python bench.py --summarise-pmc FETCH_DIR WRITE_DIR --workload NAME   (no GPU: rewrites profiles/hbm_traffic.json
                    from two rocprofv3 --pmc runs of this file)

A step is one forward plus one backward of the fused sequence+depth attention on
one batch of synthetic, HBM-resident input.  The default workload is the
long-context headline: causal, bf16, B=1, T=65536, Hq=16 (Hkv=4, G=4), D=128,
L=24; the same line carries, under ``configs``, every other benchmark configuration (c2, c3 with their plain
causal twins of the same shape, c5 and its depth-only variant).  Prints ONE JSON line.  Only the
``cpu_baseline`` leg imports ``oracle``.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (B, T, Hkv, G, D, L, mode, chunk_tokens)
    "c2": (2, 4096, 4, 4, 128, 8, "causal", 0),
    "c3": (1, 16384, 4, 4, 128, 24, "chunk_visible", 16),
    "c4": (1, 65536, 4, 4, 128, 24, "causal", 0),
    "c5": (64, 197, 6, 1, 64, 12, "noncausal", 0),
    "c5fda": (64, 197, 6, 1, 64, 12, "depth_only", 0),
    "plain": (1, 65536, 4, 4, 128, 0, "plain", 0),
    # c2 with a head dim between the matrix kernels' tile widths (runs zero-padded to 128)
    "c2d96": (2, 4096, 4, 4, 96, 8, "causal", 0),
    # c2 with head dims above 128 (the 256-wide tiles; 192 runs zero-padded)
    # the c3 token count with head dim 64 (the 64-wide tiles on a compute-bound shape)
    "c3d64": (1, 16384, 4, 4, 64, 24, "causal", 0),
    "c2d256": (2, 4096, 4, 4, 256, 8, "causal", 0),
    "c2d192": (2, 4096, 4, 4, 192, 8, "causal", 0),
    # the last block of the reference's smallest MoDA vision model (4 query heads on 1 kv head, 11 earlier layers)
    "deit_tiny": (64, 197, 1, 4, 64, 11, "noncausal", 0),
    "plain_c2": (2, 4096, 4, 4, 128, 0, "plain", 0),
    "plain_c3": (1, 16384, 4, 4, 128, 0, "plain", 0),
    # the c4 token count as one packed variable-length batch (cu_seqlens): 1 x 16K, 2 x 8K, 4 x 4K, 8 x 2K tokens
    "c4packed": (1, 65536, 4, 4, 128, 24, "causal", 0),
}
PACKED_LENGTHS = {"c4packed": [16384] + [8192] * 2 + [4096] * 4 + [2048] * 8}


def flops_fwd(B, T, Hq, D, L, mode, cb):
    if mode in ("causal", "chunk_visible", "plain"):
        pseq = T * (T + 1) // 2
    elif mode == "noncausal":
        pseq = T * T
    else:
        pseq = 0
    if L == 0:
        pdep = 0
    elif mode == "chunk_visible":
        full, rem = divmod(T, cb)
        pdep = L * (full * cb * (cb + 1) // 2 + rem * (rem + 1) // 2)
    else:
        pdep = T * L
    return 4 * D * B * Hq * (pseq + pdep)


def make_device_inputs(B, T, Hkv, G, D, L, mode, dev, seed=0):
    """Seeded N(0,1)*0.5 inputs (dO N(0,1)) generated on the device (synthetic data, bf16)."""
    import torch

    gen = torch.Generator(device=dev).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen, device=dev, dtype=torch.float32)
    qshape = (B, T, Hkv * G, D) if mode == "plain" else (B, T * G, Hkv, D)
    bf = torch.bfloat16
    q = (rn(*qshape) * 0.5).to(bf)
    k = (rn(B, T, Hkv, D) * 0.5).to(bf) if mode != "depth_only" else None
    v = (rn(B, T, Hkv, D) * 0.5).to(bf) if mode != "depth_only" else None
    kd = vd = None
    if L > 0:
        kd = torch.empty(B, T * L, Hkv, D, dtype=bf, device=dev)
        vd = torch.empty(B, T * L, Hkv, D, dtype=bf, device=dev)
        step = max(1, (T * L) // 16)
        for s in range(0, T * L, step):  # chunked to bound fp32 temporaries
            e = min(T * L, s + step)
            kd[:, s:e] = (rn(B, e - s, Hkv, D) * 0.5).to(bf)
            vd[:, s:e] = (rn(B, e - s, Hkv, D) * 0.5).to(bf)
    do = rn(*qshape).to(bf)
    return q, k, v, kd, vd, do


def bench_fp32_config(dev, steps=20):
    """The benchmark's fp32 configuration (causal, B=1, T=256, H=Hkv=4, D=64, L=4; the reference's CPU-runnable case):
    forward + backward on fp32 tensors, in exact fp32 on the vector-ALU kernels (the default) and rounded to fp16
    operands on the matrix kernels (moda_amd.set_fp32_compute("fp16"))."""
    import torch
    from moda_amd import _lib, ops

    B, T, H, D, L = 1, 256, 4, 64, 4
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=gen, device=dev, dtype=torch.float32)
    q, k, v, kd, vd, do = rn(B, T, H, D) * D ** -0.5, rn(B, T, H, D), rn(B, T, H, D), rn(B, T * L, H, D), rn(B, T * L, H, D), rn(B, T, H, D)
    out = {"workload": f"c1: causal fp32 B={B} T={T} Hq={H} Hkv={H} G=1 D={D} L={L}"}
    for setting, key in (("fp32", "ms_exact_fp32_vector_alu"), ("fp16", "ms_fp16_operands_matrix_kernels")):
        previous = ops.set_fp32_compute(setting)
        try:
            def step():
                o, lse = ops._raw_fwd(_lib.CAUSAL, q, k, v, kd, vd, 1.0, 1, 0)
                ops._raw_bwd(_lib.CAUSAL, q, k, v, kd, vd, o, lse, do, 1.0, 1, 0)
            for _ in range(3):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            out[key] = (time.perf_counter() - t0) * 1e3 / steps
        finally:
            ops.set_fp32_compute(previous)
    return out


def cpu_baseline(B, T, Hkv, G, D, L, mode, cb, target_seconds=15.0):
    """The oracle (torch restatement of the reference's naive MoDA, fp32, forward + backward) timed on the
    host cores on a bounded sample of the same workload: the LAST `tokens` tokens' query rows of ONE
    (batch, kv head) against everything they see.  Reported as TFLOP/s over the sample's algorithmic FLOPs."""
    import torch

    import oracle

    # the GPU box gives one GPU's job a share of 16 host cores whatever os.cpu_count() shows there
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    omode = "causal" if mode == "plain" else mode
    Gf = 1 if mode == "plain" else G
    inp = oracle.make_inputs(1, T, 1, D, L, Gf, seed=1, dtype=torch.float32, std=0.5,
                             depth_only=(omode == "depth_only"))

    def sample(tokens):
        t0 = T - tokens
        if omode == "chunk_visible":
            t0 = (t0 // cb) * cb
        toks = torch.arange(t0, T).repeat_interleave(Gf)
        if omode in ("causal", "chunk_visible"):
            pseq = int((toks + 1).sum())
        elif omode == "noncausal":
            pseq = toks.numel() * T
        else:
            pseq = 0
        if L == 0:
            pdep = 0
        elif omode == "chunk_visible":
            pdep = int(((toks - (toks // cb) * cb + 1) * L).sum())
        else:
            pdep = toks.numel() * L
        fl = 3.5 * 4 * D * (pseq + pdep)
        t_start = time.perf_counter()
        oracle.moda_blockwise_fwd_bwd(inp, D ** -0.5, Gf, omode, cb, block_rows=2048, token_range=(t0, T))
        return time.perf_counter() - t_start, fl, toks.numel()

    tokens = max(cb if cb else 1, min(T, 512 // Gf))
    dt, fl, nrows = sample(tokens)
    while dt < target_seconds / 3 and tokens * 2 <= T:
        tokens *= 2
        dt, fl, nrows = sample(tokens)
    return {
        "value": fl / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"last {nrows} query rows of one (batch, kv head) of the workload against all keys they see, "
                  f"oracle tiled form fp32 fwd+bwd, {dt:.2f} s of CPU time",
    }


def bench_reorg(dev, B, T, Hkv, D, L, iters=10):
    """Depth-KV reorganisation kernel at the workload's shape: L per-layer [B,T,Hkv,D] bf16 tensors ->
    token-major cache [B,T*L,Hkv,D] (one tensor; K and V each cost this).  HBM-bound: algorithmic bytes =
    read + write of B*T*L*Hkv*D*2."""
    import torch

    from moda_amd import depth_cache

    layers = [torch.randn(B, T, Hkv, D, device=dev).bfloat16() for _ in range(L)]
    cache = torch.empty(B, T * L, Hkv, D, dtype=torch.bfloat16, device=dev)
    for _ in range(2):
        depth_cache._reorg_fwd(layers, cache, 0, L)
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        depth_cache._reorg_fwd(layers, cache, 0, L)
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / iters
    nbytes = 2 * B * T * L * Hkv * D * 2
    gbs = nbytes / (ms * 1e-3) / 1e9
    out = {"kernel": "reorg_kernel", "ms": ms, "bytes": nbytes, "achieved": gbs, "unit": "GB/s",
           "peak": PEAK_HBM_GBS, "frac": gbs / PEAK_HBM_GBS, "bound": "hbm"}
    # in-place append of ONE layer into slot L-1 of the preallocated cache (what a layer costs when the
    # cache is kept and the kernels are given depth_valid, instead of the rebuild above for every layer)
    for _ in range(2):
        depth_cache._reorg_fwd(layers[:1], cache, L - 1, L)
    s.record()
    for _ in range(iters):
        depth_cache._reorg_fwd(layers[:1], cache, L - 1, L)
    e.record()
    torch.cuda.synchronize()
    ms1 = s.elapsed_time(e) / iters
    nb1 = 2 * B * T * Hkv * D * 2
    out["append_one_layer"] = {"ms": ms1, "bytes": nb1, "achieved": nb1 / (ms1 * 1e-3) / 1e9, "unit": "GB/s"}
    return out


PROBE_PATH = os.path.join(ROOT, "bench_probe.so")


def bench_mfma_probe(dev):
    """Sustained rate of a pure bf16 MFMA loop on this device, with operands drawn like the workload's
    inputs (0.5 * N(0,1), bf16) and with zeros.  The matrix pipe is power limited: random operands run
    at a lower clock than zeros, and well below the published peak, so the attention kernels' roofline
    fraction is also given against this measured ceiling.  The loop lives in ``bench_probe.so`` (built from
    ``bench_probe.hip`` by ``__graft_entry__.build()``), a benchmark-side library of its own; returns None
    when it has not been built."""
    import ctypes

    import torch

    if not os.path.exists(PROBE_PATH):
        return None
    lib = ctypes.CDLL(PROBE_PATH)
    lib.bench_probe_mfma.restype = ctypes.c_int
    lib.bench_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                     ctypes.c_void_p, ctypes.c_void_p]
    ncu = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    gen = torch.Generator().manual_seed(0)
    out = {}
    for name, tab in (("random", (0.5 * torch.randn(512 * 8, generator=gen)).bfloat16()),
                      ("zeros", torch.zeros(512 * 8, dtype=torch.bfloat16))):
        tab = tab.to(dev)
        iters = 200000  # about 30 ms: long enough for the clock to settle
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

        def launch(n):
            rc = lib.bench_probe_mfma(ctypes.c_void_p(tab.data_ptr()), n, ncu, ctypes.c_void_p(clocks.data_ptr()),
                                      ctypes.c_void_p(sink.data_ptr()), stream)
            if rc != 0:
                raise RuntimeError(f"bench_probe_mfma failed with code {rc}")

        launch(20000)
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        launch(iters)
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e)
        flop = float(ncu) * 8 * iters * 4 * 32768
        c = clocks.cpu().tolist()
        out[name] = {"tflops": flop / (ms * 1e-3) / 1e12, "shader_clock_mhz": c[0] / (c[1] / 100.0) if c[1] else None}
    return out


def bench_stack(dev, steps=10):
    """Whole-model step around the operator: the twelve blocks of the reference's smallest MoDA vision
    model (vision_tasks/deit/models.py:425-428: width 256, 4 query heads, 1 kv head, 197 tokens) at batch 64,
    bf16 weights, chained through one depth stream.  Reported: training step (forward + backward, cache rebuilt
    by the HIP reorganisation kernel), inference forward with the in-place cache, inference forward
    rebuilding the cache per layer as the reference does."""
    import torch

    import moda_amd

    torch.manual_seed(0)
    dim, depth, heads, kv_heads, B, N = 256, 12, 4, 1, 64, 197
    model = moda_amd.MoDAStack(dim, depth, heads, kv_heads).to(dev).to(torch.bfloat16)
    x = (0.5 * torch.randn(B, N, dim, device=dev)).to(torch.bfloat16)

    def train():
        model.zero_grad(set_to_none=True)
        model(x.clone().requires_grad_(True)).float().square().mean().backward()

    def infer(inplace):
        with torch.no_grad():
            model(x, inplace_cache=inplace)

    def timed(fn):
        fn()
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    return {"config": f"12 blocks, width {dim}, {heads} heads / {kv_heads} kv head, B={B}, N={N}, bf16, noncausal",
            "train_step_ms": timed(train), "inference_inplace_cache_ms": timed(lambda: infer(True)),
            "inference_rebuilt_cache_ms": timed(lambda: infer(False))}


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
# what FETCH_SIZE / WRITE_SIZE (KiB per dispatch) read for a plain copy of known size (the depth reorganisation
# kernel of the same runs): FETCH_SIZE counts half of the bytes read, WRITE_SIZE all bytes written
PMC_SCALE = {"FETCH_SIZE": 2.0, "WRITE_SIZE": 1.0}
KERNEL_NAMES = ("fwd_kernel", "fwd_wide_kernel", "delta_kernel", "dq_kernel", "dkv_kernel", "dkv_flat_kernel", "dkv_reduce_kernel", "depth_cols_kernel",
                "depth_token_handed_kernel", "depth_cols_handed_kernel", "chunk_depth_kernel", "reorg_kernel")


def depth_gradient_kernel(mode, D, G):
    """Name of the launch that forms dkd, dvd after dkv_kernel (moda_amd/csrc/geometry.h: depth_grads_in_dq,
    depth_scores_from_dq), or None where the dQ kernel forms them itself."""
    if mode == "chunk_visible":
        return "chunk_depth_kernel"
    if D <= 64 and 32 % G == 0:
        return None
    if D <= 128:
        return "depth_token_handed_kernel" if G <= 4 else "depth_cols_handed_kernel"
    return "depth_cols_kernel"


def sequence_dkv_kernel(B, T, Hkv, G, D, compute_units=256):
    """Name of the launch that forms dk, dv of the sequence keys (moda_amd/csrc/geometry.h: takes_dkv_flat,
    moda_amd/csrc/capi.hip: desired_dkv_split): short launches on the 64-wide tiles go to the kernel without the
    role split when they are short or have at least three column tiles per compute unit."""
    tiles = -(-T // 128) * B * Hkv
    split = tiles < 512 and (-(-T * G // 64)) // 2 >= 16
    return "dkv_flat_kernel" if D <= 64 and not split and (T * G <= 512 or tiles >= 3 * compute_units) else "dkv_kernel"


def recorded_traffic(workload):
    """HBM bytes per launch and kernel from profiles/hbm_traffic.json (counters cannot be read from inside this
    process: the file is rewritten by --summarise-pmc from rocprofv3 --pmc runs of this very command)."""
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)["workloads"].get(workload)
    except (OSError, ValueError, KeyError):
        return None


def summarise_pmc(fetch_dir, write_dir, workload):
    """Reads the counter_collection CSVs of `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of
    `bench.py --workload NAME --steps 1 --warmup 0 --no-cpu-baseline --no-configs` and stores, per kernel, the
    FIRST dispatch's scaled byte count (the first dispatches belong to the workload itself; the plain twin, where
    one runs, comes later with the same kernel names)."""
    import csv
    import glob

    def first_dispatch(directory, counter):
        out = {}
        files = sorted(glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True))
        if not files:
            raise SystemExit(f"no counter_collection.csv under {directory}")
        rows = []
        for fn in files:
            with open(fn) as f:
                rows += [r for r in csv.DictReader(f) if r["Counter_Name"] == counter]
        rows.sort(key=lambda r: int(r["Dispatch_Id"]))
        for r in rows:
            for kn in KERNEL_NAMES:
                if f"moda::{kn}" in r["Kernel_Name"] and kn not in out:
                    out[kn] = float(r["Counter_Value"]) * 1024.0 * PMC_SCALE[counter]
        return out

    fetch, write = first_dispatch(fetch_dir, "FETCH_SIZE"), first_dispatch(write_dir, "WRITE_SIZE")
    try:
        with open(TRAFFIC_FILE) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        doc = {}
    doc["note"] = ("HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), scaled by "
                   f"{PMC_SCALE} (what the same counters read for the reorg_kernel copy of known size); written by "
                   "`python bench.py --summarise-pmc`, read by bench.py for roofline.traffic")
    doc.setdefault("workloads", {})[workload] = {
        kn: {"fetch_bytes": fetch.get(kn, 0.0), "write_bytes": write.get(kn, 0.0),
             "bytes": fetch.get(kn, 0.0) + write.get(kn, 0.0)}
        for kn in KERNEL_NAMES if kn in fetch or kn in write}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
        f.write("\n")
    for kn, v in doc["workloads"][workload].items():
        print(f"{workload:8s} {kn:20s} read {v['fetch_bytes'] / 2**30:8.3f} GiB  written {v['write_bytes'] / 2**30:8.3f} GiB")


def min_hbm_bytes(B, T, Hkv, G, D, L, mode):
    """Every input read once and every output written once, forward + backward (bf16 tensors, fp32 statistics)."""
    es = 2
    n_q = B * T * G * Hkv * D * es
    n_kv = 0 if mode == "depth_only" else B * T * Hkv * D * es
    n_dep = B * T * L * Hkv * D * es
    n_stat = B * T * G * Hkv * 4
    fwd = n_q + 2 * n_kv + 2 * n_dep + n_q + n_stat
    bwd = 2 * n_q + 2 * n_kv + 2 * n_dep + n_q + 2 * n_stat + n_q + 2 * n_kv + 2 * n_dep + 2 * n_stat
    return fwd + bwd


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the `configs` object (the other benchmark configurations and their plain twins)")
    ap.add_argument("--with-twin", action="store_true", help="also time the plain causal twin (c4 shape, no depth)")
    ap.add_argument("--with-stack", action="store_true",
                    help="also time a 12-block attention+MLP stack chained through the depth stream")
    ap.add_argument("--summarise-pmc", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="no GPU work: rewrite profiles/hbm_traffic.json for --workload from two rocprofv3 --pmc runs")
    args = ap.parse_args()
    if args.summarise_pmc:
        summarise_pmc(args.summarise_pmc[0], args.summarise_pmc[1], args.workload)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the path shards over batch and kv heads without exchange "
              "but no multi-GPU launch is implemented. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    from moda_amd import _lib, ops

    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    def run_workload(name, steps, warmup):
        B, T, Hkv, G, D, L, mode, cb = WORKLOADS[name]
        q, k, v, kd, vd, do = make_device_inputs(B, T, Hkv, G, D, L, mode, dev)
        sc = D ** -0.5
        if mode == "plain":
            mid, Garg = _lib.PLAIN_GQA, G
        else:
            mid = {"causal": _lib.CAUSAL, "noncausal": _lib.NONCAUSAL, "chunk_visible": _lib.CHUNK_VISIBLE,
                   "depth_only": _lib.DEPTH_ONLY}[mode]
            Garg = G
        state = {}
        packed = None
        if name in PACKED_LENGTHS:
            cu = [0]
            for n_tok in PACKED_LENGTHS[name]:
                cu.append(cu[-1] + n_tok)
            assert cu[-1] == T
            packed = ops._packed(torch.tensor(cu, dtype=torch.int32, device=dev), q, G)

        def fwd():
            state["o"], state["lse"] = ops._raw_fwd(mid, q, k, v, kd, vd, sc, Garg, cb, packed=packed)

        def bwd(stages=_lib.STAGE_ALL):
            state["grads"] = ops._raw_bwd(mid, q, k, v, kd, vd, state["o"], state["lse"], do, sc, Garg, cb,
                                          stages=stages, out=state.get("grads"), ws=state.get("ws"), packed=packed)

        fwd()
        state["ws"] = ops.bwd_workspace(mid, q, k, v, kd, vd, Garg, cb, packed=packed)
        bwd()
        for _ in range(warmup):
            fwd()
            bwd()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fwd()
            bwd()
        torch.cuda.synchronize()
        ms_step = (time.perf_counter() - t0) * 1e3 / steps

        # per-kernel durations with HIP events on the launch stream (torch's current stream)
        def ev_time(fn, n):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(n):
                fn()
            e.record()
            torch.cuda.synchronize()
            return s.elapsed_time(e) / n

        n = max(2, steps // 2)
        t_fwd = ev_time(fwd, n)
        # the row sums: as a launch of their own (informational), and where a whole backward forms them, inside the
        # dQ kernel (asked for together with the dQ stage)
        t_delta = ev_time(lambda: bwd(_lib.STAGE_DELTA), n)
        t_dq = ev_time(lambda: bwd(_lib.STAGE_DELTA | _lib.STAGE_DQ), n)
        t_dkv = ev_time(lambda: bwd(_lib.STAGE_DKV), n)
        Hq = Hkv * G
        if packed is not None:
            ff = sum(flops_fwd(1, n_tok, Hq, D, L, mode, cb) for n_tok in PACKED_LENGTHS[name])
        else:
            ff = flops_fwd(B, T, Hq, D, L, mode, cb)
        return {"ms_step": ms_step, "flops_fwd": ff, "t_fwd": t_fwd, "t_delta": t_delta, "t_dq": t_dq,
                "t_dkv": t_dkv, "shape": (B, T, Hkv, G, D, L, mode, cb)}

    def describe(name, shape):
        B, T, Hkv, G, D, L, mode, cb = shape
        return (f"{name}: {mode} B={B} T={T} Hq={Hkv * G} Hkv={Hkv} G={G} D={D} L={L}"
                + (f" chunk_tokens={cb}" if cb else "")
                + (f" packed sequence lengths={PACKED_LENGTHS[name]}" if name in PACKED_LENGTHS else ""))

    def hbm_bound(shape, total_flops):
        """Small shapes (DeiT-sized c5, depth-only attention) are bound by HBM, not by the matrix pipe: reading
        every input once and writing every output once already takes longer than their FLOPs at the MFMA peak."""
        B, T, Hkv, G, D, L, mode, cb = shape
        return mode != "plain" and total_flops / min_hbm_bytes(B, T, Hkv, G, D, L, mode) \
            < PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)

    r = run_workload(args.workload, args.steps, args.warmup)
    B, T, Hkv, G, D, L, mode, cb = r["shape"]
    total_flops = 3.5 * r["flops_fwd"]
    value = total_flops / (r["ms_step"] * 1e-3) / 1e12

    # dominant kernel: dK/dV.  Algorithmic credit per backward matmul unit (one unit = flops_fwd / 2):
    # dK, dV in full plus half of the S and dP recompute it shares with the dQ kernel = 3 units;
    # the dQ kernel gets the other 2 units; forward has 2.  3 + 2 = the 5 backward units.
    unit = r["flops_fwd"] / 2
    kernels = {
        "fwd_kernel": {"ms": r["t_fwd"], "tflops": 2 * unit / (r["t_fwd"] * 1e-3) / 1e12},
        "delta_kernel": {"ms": r["t_delta"]},
        "dq_kernel": {"ms": r["t_dq"], "tflops": 2 * unit / (r["t_dq"] * 1e-3) / 1e12},
        "dkv_kernel": {"ms": r["t_dkv"], "tflops": 3 * unit / (r["t_dkv"] * 1e-3) / 1e12},
    }
    dom = max(("fwd_kernel", "dq_kernel", "dkv_kernel"), key=lambda n: kernels[n]["ms"])
    traffic = recorded_traffic(args.workload) or {}
    # the dK/dV stage is timed as a whole: dkv_kernel followed by the HBM-bound launch that forms the depth gradients
    # (where the dQ kernel does not form them itself; light launches add dkv_reduce_kernel)
    depth_kernel = depth_gradient_kernel(mode, D, G) if L > 0 else None
    two_launches = dom == "dkv_kernel" and depth_kernel is not None
    dom_traffic = None
    if dom in traffic:
        dom_traffic = traffic[dom]["bytes"]
        if dom == "dkv_kernel":
            dom_traffic += sum(traffic.get(k, {}).get("bytes", 0.0) for k in (depth_kernel, "dkv_reduce_kernel") if k)
    roofline = {
        "bound": "mfma",
        "kernel": f"dkv_kernel + {depth_kernel}" if two_launches else dom,
        "achieved": kernels[dom]["tflops"],
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": kernels[dom]["tflops"] / PEAK_BF16_TFLOPS,
        "traffic": dom_traffic,
        "traffic_source": "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, "
                          "recorded, not measured by this run)" if dom_traffic is not None else None,
    }
    if hbm_bound(r["shape"], total_flops):
        mb = min_hbm_bytes(B, T, Hkv, G, D, L, mode)
        gbs = mb / (r["ms_step"] * 1e-3) / 1e9
        whole = sum(v["bytes"] for k, v in traffic.items() if k != "reorg_kernel") if traffic else None
        launches = ["fwd_kernel", "dq_kernel"] + ([sequence_dkv_kernel(B, T, Hkv, G, D)] if mode != "depth_only" else []) \
            + ([depth_kernel] if depth_kernel else [])
        roofline = {"bound": "hbm", "kernel": " + ".join(launches),
                    "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                    "algorithmic_bytes": mb, "traffic": whole,
                    "traffic_source": "profiles/hbm_traffic.json (recorded)" if whole is not None else None}
    out = {
        "metric": "parallel_moda fwd+bwd TFLOP/s at T=64K bf16; % of bf16 MFMA peak",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": r["ms_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": describe(args.workload, r["shape"]), "flop_fwd_bwd": total_flops},
        "frac_of_bf16_mfma_peak": value / PEAK_BF16_TFLOPS,
        "kernels": kernels,
        "roofline": roofline,
    }
    if args.with_twin or args.workload == "c4":
        tw = run_workload("plain", max(2, args.steps // 2), 1)
        tw_value = 3.5 * tw["flops_fwd"] / (tw["ms_step"] * 1e-3) / 1e12
        out["plain_causal_twin"] = {"tflops": tw_value, "ms_per_step": tw["ms_step"],
                                    "moda_over_twin": value / tw_value}
    if args.workload == "c4" and not args.no_configs:
        # every other benchmark configuration in the same run: absolute rate, fraction of the matching peak,
        # per-kernel times, and for the matrix-bound ones the plain causal twin of the same shape
        configs = {}
        for name, twin in (("c2", "plain_c2"), ("c3", "plain_c3"), ("c5", None), ("c5fda", None)):
            torch.cuda.empty_cache()
            c = run_workload(name, 20, 5)
            fl = 3.5 * c["flops_fwd"]
            tf = fl / (c["ms_step"] * 1e-3) / 1e12
            entry = {"workload": describe(name, c["shape"]), "ms": c["ms_step"], "tflops": tf,
                     "frac_of_bf16_mfma_peak": tf / PEAK_BF16_TFLOPS, "flop_fwd_bwd": fl,
                     "kernel_ms": {"fwd": c["t_fwd"], "delta": c["t_delta"], "dq": c["t_dq"], "dkv": c["t_dkv"]}}
            if hbm_bound(c["shape"], fl):
                cB, cT, cH, cG, cD, cL, cmode, _ = c["shape"]
                mb = min_hbm_bytes(cB, cT, cH, cG, cD, cL, cmode)
                entry.update({"bound": "hbm", "algorithmic_bytes": mb, "gbs": mb / (c["ms_step"] * 1e-3) / 1e9,
                              "frac_of_hbm_peak": mb / (c["ms_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS})
            else:
                entry["bound"] = "mfma"
            if twin:
                t = run_workload(twin, 20, 5)
                ttf = 3.5 * t["flops_fwd"] / (t["ms_step"] * 1e-3) / 1e12
                entry["plain_causal_twin"] = {"ms": t["ms_step"], "tflops": ttf, "moda_over_twin": tf / ttf}
            configs[name] = entry
        configs["c1"] = bench_fp32_config(dev)
        out["configs"] = configs
        torch.cuda.empty_cache()
    if L > 0:
        out["depth_reorg"] = bench_reorg(dev, B, T, Hkv, D, L)
    probe = bench_mfma_probe(dev)
    if probe is not None:
        out["mfma_probe"] = probe
        out["frac_of_measured_mfma_rate"] = value / probe["random"]["tflops"]
    if args.with_stack:
        out["attention_stack"] = bench_stack(dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(B, T, Hkv, G, D, L, mode, cb)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
