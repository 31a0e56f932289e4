"""Benchmark of the map-reduce hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident in
HBM.  The default workload is the headline configuration of the reference's benchmarks: the Gaussian kernel sum
a_i = sum_j exp(-|x_i-y_j|^2/sigma^2) b_j at M = N = 1,000,000, D = 3, Dv = 1, float32.
The last line printed is ONE JSON object with the throughput (pair interactions per second), the
roofline of the dominant kernel (algorithmic flops / kernel time measured with HIP events on the
launch stream) and, for the default run, the CPU oracle timed on the host cores on a bounded sample
of the same workload.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# published MI355X peaks
PEAK_FP32_VECTOR_TFLOPS = 157.3
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_INT8_MFMA_TOPS = 5000.0
# reference number for this metric: PyKeOps Gaussian conv, M=N=1M, RTX 2080 Ti, 1.39 s
# (reference benchmarks/README.md:14) -> 7.2e11 pairs/s
PUBLISHED_PAIRS_PER_S = 1e12 / 1.39

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (summaries under profiles/);
# None until measured for a workload
MEASURED_TRAFFIC_BYTES = {
    # profiles/keops_rad_main__gauss_1m_dv1.md: FETCH_SIZE 2459909 KiB x 2.0 (copy calibration) + WRITE_SIZE 11718.75 KiB
    # (column slot vectors re-read by every row block, 98 % from L2 / Infinity Cache; 55 GB/s, not the limiter)
    "gauss_1m_dv1": int((2459909 * 2.0 + 11718.75) * 1024),
    # profiles/keops_knn_filter_i8__knn_d64.md: dominant kernel keops_knn_filter_i8 (two launches per call)
    "knn_d64": int(2 * (200093 * 2.0 + 45852) * 1024),
    # profiles/keops_chk_final__laplace_d256.md
    "laplace_d256": int((5045781 * 2.0 + 672429) * 1024),
    # profiles/keops_chk_softmax__softmax_d64.md
    "softmax_d64": int((204925 * 2.0 + 33804) * 1024),
    # profiles/keops_fin_main3__gauss_dv256.md
    "gauss_dv256": int((6304559 * 2.0 + 3617805) * 1024),
    # profiles/keops_radr_main__sparse_100x10k.md (all kernels of a launch), keops_conv_ranges__lse_b16.md
    "sparse_100x10k": int((638070 * 2.0 + 179582) * 1024),
    "lse_b16": int((55625 * 2.0 + 6250) * 1024),
    # profiles/keops_conv_dense_vchunk__knn_l1_d784.md
    "knn_l1_d784": int((4176921 * 2.0 + 39063) * 1024),
}

WORKLOADS = {
    # name: (description, algorithmic flop per pair, roofline bound)
    "gauss_1m_dv1": ("Gaussian kernel sum 1e6 x 1e6, D=3, Dv=1, float32 (benchmark configuration 2)", 14, "valu"),
    "gauss_1m_dv8": ("Gaussian kernel sum 1e6 x 1e6, D=3, Dv=8, float32 (benchmark configuration 2)", 28, "valu"),
    "gauss_1m_grad": ("gradient wrt x of the Gaussian kernel sum 1e6 x 1e6, D=3, Dv=1 (benchmark configuration 2)", 21, "valu"),
    # sum_j K_ij <e_i, b_j> (x_i - y_j) with three-component e and b (momentum-weighted gradient of shape models):
    # 12 flop of the kernel, 6 of the scalar product, 3 differences, 1 + 6 of the weighted accumulation
    "gauss_300k_grad_dv3": ("gradient wrt x of the Gaussian kernel sum 3e5 x 3e5, D=3, three weight components", 28, "valu"),
    "gauss_10k": ("Gaussian kernel sum 1e4 x 1e4, D=3, Dv=1, float32 (benchmark configuration 1)", 14, "valu"),
    "gauss_100k": ("Gaussian kernel sum 1e5 x 1e5, D=3, Dv=1, float32 (reference benchmarks/README.md:13)", 14, "valu"),
    # 2*D flop of the <x,y> contraction per pair (the matrix-core work); filter and re-rank are not counted
    # (the filter runs on signed bytes, v_mfma_i32_32x32x32_i8: the line is priced against the int8 matrix peak)
    "knn_d64": ("KMin_ArgKMin K=10, 1e5 queries x 1e6 references, D=64 (benchmark configuration 3)", 128, "mfma8"),
    # nearest neighbours among MNIST-sized rows (784 components): squared distances on the chunked matrix-core
    # sweep + exact re-rank (2*D flop of the contraction per pair), Manhattan distances on the vector-ALU chunked
    # variant of the general-purpose kernel (subtract, absolute value, add per component)
    "knn_d784": ("ArgKMin K=10 of SqDist, 1e4 queries x 6e4 references, D=784", 1568, "mfma"),
    "knn_l1_d784": ("ArgKMin K=10 of the L1 distance, 1e4 queries x 6e4 references, D=784", 2352, "valu"),
    "sparse_100x10k": ("block-sparse Gaussian sum, 100 clusters x 10,000 points (benchmark configuration 4)", 14, "valu"),
    "lse_b16": ("batched LogSumExp softmin B=16, 50,000 x 50,000, D=3 (benchmark configuration 5a)", 17, "valu"),
    # the shape of configuration 5a with a Gaussian sum instead of the log-sum-exp: batches as row ranges of the
    # matrix-core exponent kernels, one centre per batch (kernels/keops_radial_ranges.h)
    "gauss_b16": ("batched Gaussian kernel sum B=16, 50,000 x 50,000, D=3, Dv=1", 14, "valu"),
    # 2*D flop of the contraction + sqrt, neg, exp + 2*Dv of the weighted accumulation
    "laplace_d256": ("Laplace kernel sum 2e5 x 2e5, D=256, Dv=16 (benchmark configuration 5b)", 547, "mfma"),
    # softmax-weighted sum of an inner product (attention-like): 2*D flop of the scores, exp, 2*Dv of the weighted
    # sum.  Both products run on the bf16 matrix cores with float32-class accuracy (operands in two resp. three
    # bf16 terms, three resp. six instructions per block); the algorithmic flop are counted once
    "softmax_d64": ("SumSoftMaxWeight of <q,k> with 64-dimensional weights, 65536 x 65536, D=64", 258, "mfma"),
    # 12 flop of the Gaussian kernel + 2*Dv of the product with the 256-dimensional variable; the product runs on
    # the bf16 matrix cores with every operand in three bf16 terms (six instructions per block, float32 accuracy):
    # the algorithmic flop are counted once
    "gauss_dv256": ("Gaussian kernel times a 256-dimensional variable, 2e5 x 2e5, D=3 (final-product scheme)", 524, "mfma"),
}


def _np_inputs(name):
    import numpy as np

    if name.startswith("gauss_1m") or name in ("gauss_10k", "gauss_100k", "gauss_dv256", "gauss_300k_grad_dv3"):
        M = N = {"gauss_10k": 10_000, "gauss_100k": 100_000, "gauss_dv256": 200_000, "gauss_300k_grad_dv3": 300_000}.get(name, 1_000_000)
        Dv = 8 if name.endswith("dv8") else (256 if name == "gauss_dv256" else (3 if name.endswith("dv3") else 1))
        rng = np.random.default_rng(0 if name == "gauss_10k" else 1)
        x = rng.standard_normal((M, 3)).astype(np.float32)
        y = rng.standard_normal((N, 3)).astype(np.float32)
        b = rng.standard_normal((N, Dv)).astype(np.float32)
        return dict(M=M, N=N, Dv=Dv, arrays=[x, y, b, np.array([1.0], np.float32)])
    if name == "knn_d64":
        M, N, D = 100_000, 1_000_000, 64
        rng = np.random.default_rng(2)
        return dict(M=M, N=N, Dv=0, D=D, arrays=[rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)])
    if name in ("knn_d784", "knn_l1_d784"):
        M, N, D = 10_000, 60_000, 784
        rng = np.random.default_rng(7)
        return dict(M=M, N=N, Dv=0, D=D, arrays=[rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)])
    if name == "softmax_d64":
        M = N = 65_536
        rng = np.random.default_rng(6)
        q = (rng.standard_normal((M, 64)) / 64 ** 0.25).astype(np.float32)
        k = (rng.standard_normal((N, 64)) / 64 ** 0.25).astype(np.float32)
        return dict(M=M, N=N, Dv=64, D=64, arrays=[q, k, rng.standard_normal((N, 64)).astype(np.float32)])
    if name == "laplace_d256":
        M = N = 200_000
        rng = np.random.default_rng(5)
        x = (rng.standard_normal((M, 256)) / 16).astype(np.float32)
        y = (rng.standard_normal((N, 256)) / 16).astype(np.float32)
        return dict(M=M, N=N, Dv=16, D=256, arrays=[x, y, rng.standard_normal((N, 16)).astype(np.float32)])
    if name == "sparse_100x10k":
        # 100 clusters x 10,000 points N(c_k, 0.05^2), c_k ~ U[0,10)^3, sigma = 0.1, centre distance < 1 kept
        rng = np.random.default_rng(3)
        C, per = 100, 10_000
        c = (10 * rng.random((C, 3))).astype(np.float32)
        x = (np.repeat(c, per, 0) + 0.05 * rng.standard_normal((C * per, 3))).astype(np.float32)
        y = (np.repeat(c, per, 0) + 0.05 * rng.standard_normal((C * per, 3))).astype(np.float32)
        b = rng.standard_normal((C * per, 1)).astype(np.float32)
        return dict(M=C * per, N=C * per, Dv=1, centres=c, per=per, arrays=[x, y, b, np.array([100.0], np.float32)])
    if name in ("lse_b16", "gauss_b16"):
        rng = np.random.default_rng(4)
        B, M, N = 16, 50_000, 50_000
        x = rng.standard_normal((B, M, 3)).astype(np.float32)
        y = rng.standard_normal((B, N, 3)).astype(np.float32)
        l = rng.standard_normal((B, N, 1)).astype(np.float32)
        return dict(M=M, N=N, Dv=1, B=B, arrays=[x, y, l, np.array([20.0 if name == "lse_b16" else 0.5], np.float32)])
    raise SystemExit(f"workload {name} is not available in this build")


def build_step(name):
    """Returns (step callable, pairs per step, loaded module handle or None, numpy inputs)."""
    import torch

    from keops_amd.torch import Genred

    inp = _np_inputs(name)
    dev = [torch.from_numpy(a).cuda() for a in inp["arrays"]]
    M, N, Dv = inp["M"], inp["N"], inp["Dv"]
    if name == "knn_d64":
        knn = Genred("SqDist(x,y)", ["x=Vi(64)", "y=Vj(64)"], reduction_op="KMin_ArgKMin", axis=1, opt_arg=10)
        return (lambda: knn(*dev)), M * N, inp
    if name in ("knn_d784", "knn_l1_d784"):
        dist = "SqDist(x,y)" if name == "knn_d784" else "Sum(Abs(x-y))"
        knn = Genred(dist, ["x=Vi(784)", "y=Vj(784)"], reduction_op="ArgKMin", axis=1, opt_arg=10)
        return (lambda: knn(*dev)), M * N, inp
    if name == "softmax_d64":
        att = Genred("(q|k)", ["q=Vi(64)", "k=Vj(64)", "v=Vj(64)"], reduction_op="SumSoftMaxWeight", axis=1, formula2="v")
        return (lambda: att(*dev)), M * N, inp
    if name == "laplace_d256":
        lap = Genred("Exp(-Norm2(x-y))*b", ["x=Vi(256)", "y=Vj(256)", "b=Vj(16)"], reduction_op="Sum", axis=1)
        return (lambda: lap(*dev)), M * N, inp
    if name == "lse_b16":
        lse = Genred("l-SqDist(x,y)*e", ["x=Vi(3)", "y=Vj(3)", "l=Vj(1)", "e=Pm(1)"], reduction_op="LogSumExp", axis=1)
        return (lambda: lse(*dev)), inp["B"] * M * N, inp
    if name == "gauss_b16":
        gs = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)", "g=Pm(1)"], reduction_op="Sum", axis=1)
        return (lambda: gs(*dev)), inp["B"] * M * N, inp
    if name == "sparse_100x10k":
        from keops_amd.torch.cluster import from_matrix

        per, C = inp["per"], inp["centres"].shape[0]
        r = torch.tensor([[per * k, per * (k + 1)] for k in range(C)], dtype=torch.int64, device="cuda")
        ct = torch.from_numpy(inp["centres"]).cuda()
        keep = torch.cdist(ct, ct) < 1.0
        ranges = from_matrix(r, r, keep)
        sp = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)", "g=Pm(1)"], reduction_op="Sum", axis=1)
        kept_pairs = int(keep.sum().item()) * per * per  # effective pairs: kept cluster pairs only
        return (lambda: sp(*dev, ranges=ranges)), kept_pairs, inp
    conv = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", f"b=Vj({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=1)
    if name in ("gauss_1m_grad", "gauss_300k_grad_dv3"):
        # the gradient is another map-reduce (pykeops generic_red.py:165-214): run the forward once,
        # then every step back-propagates G through it, which launches the gradient kernel only
        dev[0].requires_grad_(True)
        a = conv(*dev)
        G = torch.ones_like(a) if Dv == 1 else torch.randn(a.shape, device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))

        def step():
            return torch.autograd.grad(a, [dev[0]], G, retain_graph=True)[0]
    else:
        def step():
            return conv(*dev)

    return step, M * N, inp


def kernel_modules():
    from keops_amd import keops_io

    return list(keops_io._modules.values())


def cpu_baseline(name, inp):
    """The CPU oracle (restatement of the reference's CpuReduc loop) timed on the host cores on a
    bounded sample of the same workload: a subset of output rows against all columns."""
    import numpy as np

    from oracle.cpu_oracle import cpu_reduc, lib

    M, N, Dv = inp["M"], inp["N"], inp["Dv"]
    x, y, b, g = inp["arrays"]
    lib()
    try:
        gomp = ctypes.CDLL("libgomp.so.1")
        threads = gomp.omp_get_max_threads()
    except Exception:
        gomp, threads = None, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    # calibrate on 64 rows per thread, then size the sample for about 12 s of CPU work
    ncal = int(min(M, 64 * max(1, threads)))
    rows = np.arange(ncal, dtype=np.int64)
    t0 = time.perf_counter()
    cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    rate = ncal * N / (time.perf_counter() - t0)
    nrows = int(min(M, max(256, (12.0 * rate / N) // 256 * 256)))
    rows = np.sort(np.random.default_rng(0).choice(M, nrows, replace=False)).astype(np.int64)
    t0 = time.perf_counter()
    cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    dt = time.perf_counter() - t0
    res = dict(value=nrows * N / dt, unit="pairs/s", cores=int(threads), kind="port", cpu_model=model,
               sample=f"{nrows} random output rows x {N} columns of the same inputs ({dt:.1f} s, OpenMP over rows)")
    if gomp is not None and threads > 1:
        # the same loop on one thread (about 4 s)
        n1 = int(max(16, (4.0 * rate / threads / N) // 16 * 16))
        gomp.omp_set_num_threads(1)
        t0 = time.perf_counter()
        cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows[:n1])
        dt1 = time.perf_counter() - t0
        gomp.omp_set_num_threads(int(threads))
        res["value_1_thread"] = min(n1, len(rows)) * N / dt1
        res["sample_1_thread"] = f"{min(n1, len(rows))} of those rows on one thread ({dt1:.1f} s)"
    return res


def cpu_baseline_config1():
    """The oracle on the reference's own CPU-runnable case in full (benchmark configuration 1: Gaussian sum, M = N =
    10,000, D = 3): median of 5 calls after one warm-up, on all host threads and on one."""
    import numpy as np

    from oracle.cpu_oracle import cpu_reduc

    inp = _np_inputs("gauss_10k")
    M, N, Dv = inp["M"], inp["N"], inp["Dv"]

    def median_time():
        cpu_reduc("gauss", inp["arrays"], M, N, Dv)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            cpu_reduc("gauss", inp["arrays"], M, N, Dv)
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    res = {"workload": WORKLOADS["gauss_10k"][0]}
    try:
        gomp = ctypes.CDLL("libgomp.so.1")
        threads = int(gomp.omp_get_max_threads())
    except Exception:
        gomp, threads = None, None
    t_all = median_time()
    res.update(value=M * N / t_all, unit="pairs/s", cores=threads, seconds=t_all)
    if gomp is not None and threads and threads > 1:
        gomp.omp_set_num_threads(1)
        t1 = median_time()
        gomp.omp_set_num_threads(threads)
        res.update(value_1_thread=M * N / t1, seconds_1_thread=t1)
    return res


def calibration(mfma):
    """Issue rates of loop-only kernels (keops_hip_calibrate): wavefront instructions per cycle and SIMD at the
    nominal 2.4 GHz clock, for 1, 2 and 4 wavefronts per SIMD (256 CUs x 4 SIMDs; a workgroup is 4 wavefronts)."""
    import torch

    from keops_amd import binder

    cus = torch.cuda.get_device_properties(0).multi_processor_count
    simds, clock = 4 * cus, 2.4e9
    rows = []
    kinds = [(3, "v_mfma_f32_32x32x16_bf16", (1, 2, 4)), (4, "v_mfma_f32_32x32x16_f16", (1, 2, 4)),
             (6, "v_mfma_i32_32x32x32_i8", (1, 2, 4)),
             (7, "two chains, operands change with every instruction (chains = 0: bf16, 1: f16, 2: i8)", (0, 1, 2)),
             (8, "byte filter loop without memory traffic: 4 v_mfma_i32_32x32x32_i8 and two 16-value minima per round "
                 "(chains = 0: minima over the results, 1: over other registers, 2: no minima)", (2, 1, 0)),
             (9, "contraction loop of the chunked kernel alone: hi/lo half-precision rows in registers, tiles streamed "
                 "through LDS, 48 v_mfma_f32_32x32x16_f16 per round (chains = 0: constant operands, 1: random)", (0, 1)),
             (5, "two chains of v_mfma_f32_32x32x16_bf16 with `chains` v_fmac_f32 after every matrix instruction", (0, 1, 2, 4, 8))] if mfma else [
        (0, "v_fmac_f32 chains", (1, 2, 4, 8)), (1, "Gaussian pair mix with v_exp_f32 (9 instr)", (1, 2, 4, 8)),
        (2, "Gaussian pair mix without v_exp_f32 (8 instr)", (1, 2, 4, 8)),
        (10, "Gaussian pair, every operation rounded on its own (12 instr), `chains` pairs advanced statement by statement",
         (1, 2, 4)),
        (11, "written-out sequences, 8 wavefronts per SIMD (chains = sequence: 0 v_mul vgpr, 1 v_mul sgpr operand, 2 v_mul "
             "literal, 3 v_add, 4 v_fmac, 5 v_fma three registers, 6 v_max, 7 v_perm_b32, 8 v_exp_f32, 9 v_exp_f32 alternating "
             "with v_fmac, 10 rounded Gaussian pair (12 instr), 11 contracted pair (9 instr), 12 v_max3)", tuple(range(13))),
        (12, "stream of the Gaussian sweep alone: 4 v_mfma_f32_32x32x16_bf16 per 32 pairs, v_exp_f32 and `chains` v_fmac_f32 "
             "per pair; the rate counts pairs (v_exp_f32)", (1, 4, 8))]
    for kind, label, chain_set in kinds:
        for chains in chain_set:
            # one workgroup = 4 wavefronts = one per SIMD of a CU (kind 9: 8 wavefronts, at most two workgroups per CU)
            wg_waves = 8 if kind in (9, 12) else 4
            for wgs in ((1, 2) if kind in (9, 12) else (8,) if kind == 11 else (1, 2, 4)):
                blocks, waves = cus * wgs, wgs * wg_waves // 4
                iters = {7: 12_500, 8: 100_000, 5: 50_000, 9: 4_000, 11: 20_000, 12: 20_000}.get(kind) or (200_000 if kind < 3 or kind == 10 else 100_000) // chains
                ms, ipw = binder.calibrate(kind, chains, blocks, iters)
                total = ipw * blocks * wg_waves  # wavefront instructions
                per_cycle = total / (ms * 1e-3) / simds / clock
                row = dict(kind=label, chains=chains, waves_per_simd=waves, ms=round(ms, 3),
                           wave_instr_per_cycle_per_simd_at_2p4GHz=round(per_cycle, 4))
                if 3 <= kind <= 9:
                    # (kind 6: integer operations, 32 x 32 x 32 per instruction)
                    depth = 32 if kind in (6, 8) or (kind == 7 and chains == 2) else 16
                    row["PFLOP_per_s"] = round(total * 32 * 32 * depth * 2 / (ms * 1e-3) / 1e15, 3)
                else:
                    row["lane_instr_per_s"] = total * 64 / (ms * 1e-3)
                    row["ns_per_wave_instr_and_simd"] = round(ms * 1e6 / (total / simds), 4)
                rows.append(row)
    return {"calibration": "mfma" if mfma else "valu", "cus": cus, "rows": rows}


# the other targets of the hot path: reported beside the headline line so that one default run shows all of them
SIDE_WORKLOADS = ["gauss_1m_dv8", "gauss_1m_grad", "knn_d64", "sparse_100x10k", "lse_b16", "laplace_d256"]


def measure(workload, steps, warmup):
    """Times `steps` passes of one workload (after `warmup` untimed ones, synchronised on both sides) and the main
    kernels of a pass between HIP events on the launch stream."""
    import torch

    desc, flop_per_pair, bound = WORKLOADS[workload]
    before = set(id(m) for m in kernel_modules())
    step, pairs, inp = build_step(workload)
    for _ in range(max(1, warmup)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps

    # kernel-only time: HIP events recorded by the library around the launch, on the launch stream; only the
    # modules this workload loaded are asked.  Taken right behind the timed steps, so that both figures see the same
    # clocks (a pass that waits for its events after a pause runs up to a tenth slower on the short workloads)
    mods = [m for m in kernel_modules() if id(m) not in before] or kernel_modules()
    for m in mods:
        m.set_timing(True)
    kernel_ms = []
    for _ in range(min(3, steps)):
        step()
        kernel_ms.append(max(m.last_kernel_ms() for m in mods))
    for m in mods:
        m.set_timing(False)
    torch.cuda.synchronize()

    kms = sum(kernel_ms) / len(kernel_ms)
    achieved = pairs * flop_per_pair / (kms * 1e-3) / 1e12
    peak = {"valu": PEAK_FP32_VECTOR_TFLOPS, "mfma": PEAK_BF16_MFMA_TFLOPS, "mfma32": PEAK_FP32_MFMA_TFLOPS,
            "mfma8": PEAK_INT8_MFMA_TOPS}[bound]
    note = {"valu": "peak is the packed-FP32 vector figure; packed FP32 instructions are disabled in this build. "
                    "Gaussian sums take their exponents from the matrix cores when the device-side check allows it "
                    "(kernels/keops_radial_mfma.h): the vector ALU then issues v_exp_f32 + one fma per pair and output "
                    "component, and the algorithmic flop of the exponent are not vector-ALU work any more",
            "mfma": "peak is the dense bf16 matrix figure", "mfma32": "peak is the dense fp32 matrix figure",
            "mfma8": "peak is the dense int8 matrix figure (5.0 POP/s): the fixed-threshold filter runs on signed bytes when "
                     "the device finds the quantisation slack small against the search radii (kernels/keops_knn_mfma.h, "
                     "keops_knn_filter_i8); with KEOPS_AMD_KNN_I8=0 the same call runs its filter in bfloat16 "
                     "(12.7 ms, 0.40 of the 2.5 PFLOP/s bf16 peak).  `achieved` counts the 2*D operations of <x,y> per "
                     "pair once; sampling pass and exact re-rank are not counted"}[bound]
    return dict(desc=desc, flop_per_pair=flop_per_pair, bound=bound, pairs=pairs, inp=inp, dt=dt, kernel_ms=kms,
                achieved=achieved, peak=peak, note=note)


def side_configs(steps=3, warmup=2):
    """{workload: {ms, kernel_ms, pairs_per_s, frac, bound, peak}} for the other targets of the hot path, a few steps each."""
    import gc

    import torch

    res = {}
    for name in SIDE_WORKLOADS:
        r = measure(name, steps, warmup)
        res[name] = {"workload": r["desc"], "ms": r["dt"] * 1e3, "kernel_ms": r["kernel_ms"], "pairs_per_s": r["pairs"] / r["dt"],
                     "achieved": r["achieved"], "peak": r["peak"], "unit": "TFLOP/s" if r["bound"] != "mfma8" else "TOP/s",
                     "frac": r["achieved"] / r["peak"], "bound": "mfma" if r["bound"].startswith("mfma") else r["bound"],
                     "flop_per_pair": r["flop_per_pair"], "steps": steps}
        del r
        gc.collect()
        torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="gauss_1m_dv1", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-side-configs", action="store_true",
                    help="default workload only: skip the short runs of the other targets (the `configs` object of the line)")
    ap.add_argument("--valu-calibration", action="store_true",
                    help="loop-only kernels: what the vector ALU sustains on chains of v_fmac_f32 and on the "
                         "instruction mix of a Gaussian pair, with and without v_exp_f32, at 1/2/4 wavefronts per SIMD")
    ap.add_argument("--mfma-calibration", action="store_true",
                    help="loop-only kernels: what the matrix cores sustain on 1/2/4 dependent chains of "
                         "v_mfma_f32_32x32x16_bf16 per wavefront")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run a plain 1 GiB device copy instead of a workload (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a HIP device")
    if args.valu_calibration or args.mfma_calibration:
        print(json.dumps(calibration(args.mfma_calibration)))
        return
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4, "copies": args.steps}))
        return
    r = measure(args.workload, args.steps, args.warmup)
    desc, flop_per_pair, bound, pairs, inp, dt, kms, achieved, peak, note = (
        r["desc"], r["flop_per_pair"], r["bound"], r["pairs"], r["inp"], r["dt"], r["kernel_ms"], r["achieved"], r["peak"], r["note"])
    out = {
        "metric": "pair interactions/sec (M*N/s), 1e6x1e6 D=3 Gauss sum" if args.workload == "gauss_1m_dv1"
        else "pair interactions/sec (M*N/s)",
        "value": pairs / dt,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": (pairs / dt) / PUBLISHED_PAIRS_PER_S if args.workload == "gauss_1m_dv1" else None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": desc, "M": inp["M"], "N": inp["N"], "D": inp.get("D", 3), "Dv": inp["Dv"],
                   "baseline_hardware": "RTX 2080 Ti (reference benchmarks/README.md:14)"},
        "roofline": {
            "bound": "mfma" if bound.startswith("mfma") else bound, "achieved": achieved, "peak": peak, "unit": "TFLOP/s", "frac": achieved / peak,
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
            "kernel_ms": kms, "end_to_end_ms": dt * 1e3, "flop_per_pair": flop_per_pair,
            "note": note,
        },
    }
    if args.workload == "gauss_1m_dv1" and not args.no_side_configs:
        del r, inp
        out["configs"] = side_configs()
    if args.workload == "gauss_1m_dv1" and not args.no_cpu_baseline:
        inp = _np_inputs(args.workload)
        out["cpu_baseline"] = cpu_baseline(args.workload, inp)
        out["cpu_baseline"]["config1"] = cpu_baseline_config1()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
