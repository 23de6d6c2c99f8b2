#!/usr/bin/env python3
"""Benchmark of the fused pseudorandom-matrix linear layer (forward + both backward products) on one MI355X.

Workload (the configuration the headline metric is quoted on): one layer at the GPT-2 small MLP up-projection
shape, in = 768 -> out = 3072, coef dim k = 256 (matrix-coef, C is [3072 x 256]), 8192 tokens, bf16
activations with fp32 accumulation, x ~ N(0,1), dy ~ N(0,1), C ~ N(0, 3*0.02^2/k), seed 0.  Synthetic data.

A "step" is one pass of the hot path, y = x W^T, dx = dy W, dC = (dy^T x) N^T with W = C N never stored, through
the C ABI of librandumb_hip.so with inputs already resident in HBM, the way a training step calls it:
  forward   rdb_linear_project (z = x N^T, kept for the backward pass in place of x) + rdb_linear_fwd_projected
  backward  rdb_linear_bwd_projected (dx and dC from dy, z, C in two launches)
The printed JSON line reports
  value        algorithmic TFLOP/s of the whole step, F = 6*T*in*out + 6*out*in*k (three dense products plus the
               weight generation per direction and the dC contraction).  The kernels use W = C N associatively and
               execute fewer flops than F (config.executed_gflop_per_step); both figures are printed.
  roofline     the backward call (two thirds of F, the slowest call) against the dense bf16 MFMA peak, from HIP events
  cpu_baseline the CPU restatement (materialise-then-matmul: oracle C + torch.matmul fp32) on the host cores
  compare      the one-call entry points (z recomputed in the backward pass), the kernels that do form W tiles on
               chip, materialise-to-HBM + dense GEMM on the GPU, and a plain dense GEMM
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

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
# HBM bytes per call of each product, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this script scaled by what the same
# counters read for a plain 256 MiB device copy (FETCH x2.000, WRITE x1.000): profiles/bench_c2_hbm_traffic.md
HBM_TRAFFIC_BYTES = {
    "forward (factored_z_kernel + factored_ys_kernel)": 84.2e6,
    "backward (bwd_dc_dyc_kernel + bwd_tns_red_kernel)": 144.1e6 + 35.8e6,
}
T, IN_F, OUT_F, K, SEED = 8192, 768, 3072, 256, 0


F_PER_PRODUCT = 2.0 * T * IN_F * OUT_F + 2.0 * OUT_F * IN_F * K      # one dense product + one W generation / dC contraction
F_STEP = 3.0 * F_PER_PRODUCT
# what the factored kernels execute: z, y, t, dx, dC products (z once per step)
EXEC = {
    "forward (factored_z_kernel + factored_ys_kernel)": 2.0 * T * K * (IN_F + OUT_F),
    "backward (bwd_dc_dyc_kernel + bwd_tns_red_kernel)": 2.0 * T * K * (OUT_F + IN_F) + 2.0 * T * K * OUT_F,
}
EXEC_STEP = 2.0 * T * K * (IN_F + OUT_F) + 2.0 * T * K * (OUT_F + IN_F) + 2.0 * T * K * OUT_F


def other_configs(event_ms):
    """The other two single-layer configurations, timed for the record (they are parity-test cases, not the metric)."""
    import torch

    from randumb_amd import hip

    out = {}
    # small-k fp32 regime: 4096 -> 4096, k = 16, forward at batch 1 / 16 / 256.  "effective" = the bytes a stored-W product
    # would move (4*(out*in + B*in + B*out)) over the time; the fused kernel itself reads 4*(B*in + out*k) and writes 4*B*out.
    in_f = out_f = 4096
    g = torch.Generator().manual_seed(0)
    C = (torch.randn(out_f, 16, generator=g) / 64.0).cuda()
    small = {}
    import ctypes

    from randumb_amd import _lib
    L = _lib.load()
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    for B in (1, 16, 256):
        x = torch.randn(B, in_f, generator=g).cuda()
        y = torch.empty(B, out_f, device="cuda")
        d = _lib.LinearDesc()
        d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = B, in_f, out_f, 16, out_f, in_f, 1, 0
        d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_F32, _lib.RDB_F32, _lib.RDB_ALGO_AUTO
        r = ctypes.byref(d)
        n = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, r)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device="cuda")
        args = (vp(y.data_ptr()), out_f, vp(x.data_ptr()), in_f, vp(C.data_ptr()), None, None, r, vp(ws.data_ptr()), n, stream)
        _lib.check(L.rdb_linear_fwd(*args), "rdb_linear_fwd")
        ms = event_ms(lambda: L.rdb_linear_fwd(*args), 200)   # two tiny launches per call: bounded by the host's launch rate
        stored = 4.0 * (out_f * in_f + B * in_f + B * out_f)
        actual = 4.0 * (B * in_f + out_f * 16 + B * out_f)
        small[f"batch_{B}"] = {"fwd_ms": round(ms, 4), "effective_GBps_vs_stored_W": round(stored / ms / 1e6, 1),
                               "actual_HBM_GBps": round(actual / ms / 1e6, 2)}
    out["in4096_out4096_k16_fp32_matrix_coef"] = small
    # LLM-sized layer: 4096 -> 14336, k = 1024, 4096 tokens, bf16, forward + backward through the projected entry points
    T, in_f, out_f, k = 4096, 4096, 14336, 1024
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda()
    dy = torch.randn(T, out_f, generator=g).bfloat16().cuda()
    C = (torch.randn(out_f, k, generator=g) / 64.0 * (3.0 / k) ** 0.5).bfloat16().cuda()

    def step():
        z = hip.linear_project(x, k, out_f, 0, coef=C)
        hip.linear_fwd_projected(z, C, in_f, 0)
        hip.linear_bwd_projected(dy, z, C, in_f, 0)

    ms = event_ms(step, 10)
    F = 6.0 * T * in_f * out_f + 6.0 * out_f * in_f * k
    executed = 4.0 * T * k * (in_f + out_f) + 2.0 * T * k * out_f
    out["in4096_out14336_k1024_T4096_bf16"] = {"fwd_bwd_ms": round(ms, 4), "algorithmic_TFLOPs": round(F / ms / 1e9, 1),
                                               "frac_of_mfma_peak": round(F / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                                               "executed_TFLOPs": round(executed / ms / 1e9, 1),
                                               "note": "includes torch allocation of outputs and workspace per call"}
    # GPT-2 small with random-backed linears: 12 layers, d = 768, 12 heads, vocab 50304, k = 256, seeds 0..47, bf16,
    # batch 8 x 1024 random token ids; one training step (forward + backward).  Attention, norms, embedding, head and loss
    # are stock PyTorch; the 48 linears run the projected kernels.
    from randumb_amd.SillyLayers import listgen, stepgen
    from randumb_amd.gpt import RT_GPT, RT_GPTConfig

    torch.manual_seed(0)
    model = RT_GPT(RT_GPTConfig(int_dim_gen=listgen([256] * 48), seed_gen=stepgen(0, 1))).to(torch.bfloat16).cuda()
    idx = torch.randint(0, 50304, (8, 1024), generator=g).cuda()
    tgt = torch.randint(0, 50304, (8, 1024), generator=g).cuda()

    def gpt_step():
        model.zero_grad(set_to_none=True)
        model(idx, tgt).backward()

    ms = event_ms(gpt_step, 5)
    out["gpt2_small_12L_k256_seeds0to47_bf16_8x1024"] = {"fwd_bwd_ms": round(ms, 2), "tokens_per_s": round(8192 / ms * 1e3, 0),
                                                        "note": "random-backed qkv/proj/fc/mlp-proj; attention, norms, embedding, "
                                                                "head and loss are stock PyTorch"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--no-compare", action="store_true", help="skip the materialise+GEMM comparison legs")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch plain device copies of 256 MiB (a known 256 MiB read + 256 MiB written per launch) so that "
                         "hardware byte counters collected over this run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from randumb_amd import _lib, hip

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = _lib.load()

    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, IN_F, generator=g).bfloat16().to(dev)
    dy = torch.randn(T, OUT_F, generator=g).bfloat16().to(dev)
    C = (torch.randn(OUT_F, K, generator=g) * (3 * 0.02**2 / K) ** 0.5).bfloat16().to(dev)
    y = torch.empty(T, OUT_F, dtype=torch.bfloat16, device=dev)
    dx = torch.empty(T, IN_F, dtype=torch.bfloat16, device=dev)
    dC = torch.empty(OUT_F, K, dtype=torch.float32, device=dev)

    d = _lib.LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows = T, IN_F, OUT_F, K, OUT_F
    d.sO, d.sI, d.seed = IN_F, 1, SEED
    d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_BF16, _lib.RDB_BF16, _lib.RDB_ALGO_AUTO
    dref = ctypes.byref(d)
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    px, pdy, pC, py, pdx, pdC = (vp(t.data_ptr()) for t in (x, dy, C, y, dx, dC))

    # caller-owned scratch, sized by the library (nothing is allocated inside the timed region)
    ws_bytes = max(L.rdb_linear_workspace_bytes(op, dref) for op in (_lib.RDB_OP_LINEAR_FWD, _lib.RDB_OP_LINEAR_BWD_DX,
                                                                     _lib.RDB_OP_LINEAR_BWD_DCOEF, _lib.RDB_OP_LINEAR_BWD_PROJECTED))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    pws = vp(ws.data_ptr())
    z_bytes = L.rdb_linear_projection_bytes(dref)
    assert z_bytes > 0, "the projected form must apply to the headline workload"
    z = torch.empty(z_bytes, dtype=torch.uint8, device=dev)   # the projection state: z in two orders and C transposed
    pz = vp(z.data_ptr())

    def k_project():
        _lib.check(L.rdb_linear_project(pz, px, IN_F, pC, dref, stream), "rdb_linear_project")

    def k_fwd_projected():
        _lib.check(L.rdb_linear_fwd_projected(py, OUT_F, pz, pC, None, dref, stream), "rdb_linear_fwd_projected")

    def k_dx():
        _lib.check(L.rdb_linear_bwd_dx(pdx, IN_F, pdy, OUT_F, pC, None, dref, pws, ws_bytes, stream), "rdb_linear_bwd_dx")

    def k_dcoef_projected():
        _lib.check(L.rdb_linear_bwd_dcoef_projected(pdC, pdy, OUT_F, pz, dref, stream), "rdb_linear_bwd_dcoef_projected")

    def k_fwd():
        k_project()
        k_fwd_projected()

    def k_bwd():
        _lib.check(L.rdb_linear_bwd_projected(pdx, IN_F, pdC, pdy, OUT_F, pz, pC, dref, pws, ws_bytes, stream), "rdb_linear_bwd_projected")

    def step():
        k_fwd()
        k_bwd()

    # the one-call entry points: the same kernels, z recomputed into the workspace by the coefficient gradient
    def make_onecall(algo):
        dd = _lib.LinearDesc.from_buffer_copy(d)
        dd.algo = algo
        r = ctypes.byref(dd)

        def fwd():
            _lib.check(L.rdb_linear_fwd(py, OUT_F, px, IN_F, pC, None, None, r, pws, ws_bytes, stream), "rdb_linear_fwd")

        def dxf():
            _lib.check(L.rdb_linear_bwd_dx(pdx, IN_F, pdy, OUT_F, pC, None, r, pws, ws_bytes, stream), "rdb_linear_bwd_dx")

        def dcf():
            _lib.check(L.rdb_linear_bwd_dcoef(pdC, None, pdy, OUT_F, px, IN_F, r, pws, ws_bytes, stream), "rdb_linear_bwd_dcoef")

        return fwd, dxf, dcf, dd

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    F = F_STEP
    value = F / (ms_per_step * 1e-3) / 1e12

    # per-call durations from HIP events recorded on the stream the kernels are launched on
    def event_ms(fn, iters):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    # spread of single steps, each between its own pair of events (as triton's do_bench reports: median, 20th, 80th percentile)
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    evs[0].record()
    for i in range(args.steps):
        step()
        evs[i + 1].record()
    torch.cuda.synchronize()
    per_step = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps))
    pct = lambda q: per_step[min(len(per_step) - 1, int(q * len(per_step)))]
    step_spread = {"p20": round(pct(0.2), 5), "p50": round(pct(0.5), 5), "p80": round(pct(0.8), 5)}

    iters = max(10, min(args.steps, 50))
    calls = {
        "rdb_linear_project": event_ms(k_project, iters),
        "rdb_linear_fwd_projected": event_ms(k_fwd_projected, iters),
        "rdb_linear_bwd_projected": event_ms(k_bwd, iters),
        "rdb_linear_bwd_dx (separate call)": event_ms(k_dx, iters),
        "rdb_linear_bwd_dcoef_projected (separate call)": event_ms(k_dcoef_projected, iters),
    }
    products = {   # share of F: forward one third, backward (dx and dC) two thirds
        "forward (factored_z_kernel + factored_ys_kernel)": (calls["rdb_linear_project"] + calls["rdb_linear_fwd_projected"], F_PER_PRODUCT),
        "backward (bwd_dc_dyc_kernel + bwd_tns_red_kernel)": (calls["rdb_linear_bwd_projected"], 2 * F_PER_PRODUCT),
    }
    dom = max(products, key=lambda n: products[n][0])
    dom_ms, dom_flops = products[dom]
    achieved = dom_flops / (dom_ms * 1e-3) / 1e12
    roofline = {
        "bound": "mfma", "kernel": dom, "achieved": round(achieved, 3), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 5), "traffic": HBM_TRAFFIC_BYTES[dom], "avg_kernel_ms": round(dom_ms, 5),
        "algorithmic_gflop_per_launch": round(dom_flops / 1e9, 3),
        "executed_gflop_per_launch": round(EXEC[dom] / 1e9, 3), "executed_frac": round(EXEC[dom] / (dom_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 5),
        "calls_ms": {n: round(v, 5) for n, v in calls.items()},
    }

    compare = None
    if not args.no_compare:
        def mat_gemm_step():
            # the reference's data flow on the GPU: W to HBM (twice per step), three dense GEMMs, dW to HBM
            W = hip.materialize_fwd(C, (OUT_F, IN_F), (IN_F, 1), SEED, None, False).to(torch.bfloat16)
            yy = x @ W.t()
            W2 = hip.materialize_fwd(C, (OUT_F, IN_F), (IN_F, 1), SEED, None, False).to(torch.bfloat16)
            dxx = dy @ W2
            dW = dy.t() @ x
            dCC = hip.materialize_bwd(dW, K, SEED, coef_rows=OUT_F)
            return yy, dxx, dCC

        Wd = torch.randn(OUT_F, IN_F, device=dev).bfloat16()

        def dense_step():
            return x @ Wd.t(), dy @ Wd, dy.t() @ x

        def vendor_skinny():
            # the three dense products of the factored algorithm given to the vendor GEMM (torch.matmul), for reference
            # against factored_ys_kernel / dx_dyc_kernel / factored_dc_kernel in profiles/bench_c2_kernel_trace.md
            zz = torch.randn(T, K, device=dev).bfloat16()
            yy = torch.empty(T, OUT_F, device=dev, dtype=torch.bfloat16)
            tt = torch.empty(T, K, device=dev, dtype=torch.bfloat16)
            cc = torch.empty(OUT_F, K, device=dev, dtype=torch.bfloat16)
            return {"y = z.C^T": round(event_ms(lambda: torch.matmul(zz, C.t(), out=yy), 30), 4),
                    "t = dy.C": round(event_ms(lambda: torch.matmul(dy, C, out=tt), 30), 4),
                    "dC = dy^T.z": round(event_ms(lambda: torch.matmul(dy.t(), zz, out=cc), 30), 4)}

        def onecall_ms(algo):
            fwd, dxf, dcf, _keep = make_onecall(algo)
            return {"fwd": round(event_ms(fwd, 20), 4), "dx": round(event_ms(dxf, 20 if algo != _lib.RDB_ALGO_TILE else 3), 4),
                    "dcoef": round(event_ms(dcf, 20), 4)}

        def strip_ms():
            # the algorithm that does form W, never in HBM: forward strip, dx from a noise strip kept in LDS, dcoef from dW tiles
            t = onecall_ms(_lib.RDB_ALGO_STRIP)
            return {"fwd_strip": t["fwd"], "dx_noise_strip": t["dx"], "dcoef_dw_tile": t["dcoef"],
                    "step": round(t["fwd"] + t["dx"] + t["dcoef"], 4), "dx_tile": onecall_ms(_lib.RDB_ALGO_TILE)["dx"]}

        compare = {
            "one_call_entry_points_ms": onecall_ms(_lib.RDB_ALGO_AUTO),
            "w_tiles_formed_on_chip_ms": strip_ms(),
            "vendor_gemm_on_the_factored_shapes_ms": vendor_skinny(),
            "materialize_then_gemm_ms": round(event_ms(mat_gemm_step, 10), 4),
            "dense_gemm_only_ms": round(event_ms(dense_step, 20), 4),
        }

    other = None
    if not args.no_compare:
        other = other_configs(event_ms)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import oracle

        oracle.build()
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        os.environ.setdefault("OMP_NUM_THREADS", "16")
        xc, dyc, Cc = x.float().cpu(), dy.float().cpu(), C.float().cpu().numpy()

        def cpu_step():
            W = torch.from_numpy(oracle.materialize_fwd(Cc, (OUT_F, IN_F), (IN_F, 1), SEED, row_len=IN_F, acc_double=False))
            yy = xc @ W.t()
            W2 = torch.from_numpy(oracle.materialize_fwd(Cc, (OUT_F, IN_F), (IN_F, 1), SEED, row_len=IN_F, acc_double=False))
            dxx = dyc @ W2
            dW = dyc.t() @ xc
            dCC = oracle.materialize_bwd(dW.numpy(), K, SEED, coef_rows=OUT_F)
            return yy, dxx, dCC

        cpu_step()  # warm-up
        n_cpu = 3
        c0 = time.perf_counter()
        for _ in range(n_cpu):
            cpu_step()
        c_ms = (time.perf_counter() - c0) * 1e3 / n_cpu
        cpu_baseline = {
            "value": round(F / (c_ms * 1e-3) / 1e12, 5), "unit": "TFLOP/s", "cores": int(oracle.lib().rdbo_num_threads()),
            "kind": "port", "ms_per_step": round(c_ms, 2),
            "sample": f"{n_cpu} full fwd+bwd steps of the same workload, fp32: oracle C materialise (OpenMP) + torch.matmul",
        }

    out = {
        "metric": "fused PRNG-GEMM fwd+bwd TFLOP/s & % MFMA peak at 768->3072,k=256,8192 tok",
        "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "single fused layer 768->3072, k=256 matrix-coef, 8192 tokens, bf16 act / fp32 accumulate, fwd+dx+dcoef",
                   "tokens": T, "in": IN_F, "out": OUT_F, "k": K, "seed": SEED, "algorithmic_gflop_per_step": round(F / 1e9, 3),
                   "executed_gflop_per_step": round(EXEC_STEP / 1e9, 3), "executed_tflops": round(EXEC_STEP / (ms_per_step * 1e-3) / 1e12, 3),
                   "algorithm": "factored: y=(x N^T) C^T, dx=(dy C) N, dC=dy^T (x N^T); z = x N^T computed once per step"},
        "frac_of_mfma_peak": round(value / MFMA_BF16_PEAK_TFLOPS, 5),
        "ms_per_step_events": step_spread,
        "roofline": roofline, "cpu_baseline": cpu_baseline, "compare": compare, "other_configs": other,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
