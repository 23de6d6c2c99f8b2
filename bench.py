#!/usr/bin/env python3
"""Benchmark of the fused pseudorandom-matrix linear layer (forward + both backward products) on one MI355X.

Workload (the configuration the headline metric is quoted on): one layer at the GPT-2 small MLP up-projection
shape, in = 768 -> out = 3072, coef dim k = 256 (matrix-coef, C is [3072 x 256]), 8192 tokens, bf16
activations with fp32 accumulation, x ~ N(0,1), dy ~ N(0,1), C ~ N(0, 3*0.02^2/k), seed 0.  Synthetic data.

A "step" is one pass of the hot path, y = x W^T, dx = dy W, dC = (dy^T x) N^T with W = C N never stored, through
the C ABI of librandumb_hip.so with inputs already resident in HBM, the way a training step calls it:
  forward   rdb_linear_project_fwd (z = x N^T and the transposed coefficients, kept for the backward pass,
            and y = z C^T, in one launch)
  backward  rdb_linear_bwd_projected (dx and dC from dy, the projection state and C, in two launches)
Every buffer (inputs, outputs, projection state, workspace) is allocated before the timed region.

What the printed JSON line says, and with which clock:
  ms_per_step            host clock (time.perf_counter) around exactly --steps steps, a device synchronisation on both sides,
                         every step on the SAME buffers: about 150 MB per step, which the 256 MB last-level cache holds from
                         one step to the next.  A step is three launches of 10 to 40 us; Python may issue them more slowly than
                         the GPU runs them, so the step is recorded into a HIP graph once and a timed step is one replay
                         (ms_per_step_graph); ms_per_step_eager is the same loop with the two C-ABI calls issued one by one.
                         ms_per_step is the smaller of the two and `launch` says which
  ms_per_step_rotating   the same loop over 3 buffer sets in turn (480 MB: nothing a step reads is left in a cache by the
                         step before): the number to expect inside a real training step
  ms_per_step_events     HIP events on the launch stream: one pair around all steps ("all"), and median / 20th / 80th
                         percentile of single steps each between its own pair (the extra event records between steps make
                         these a few microseconds longer than the host-clock figure)
  value                  F / ms_per_step with F = 6*T*in*out + 6*out*in*k, the flops of the algorithm the metric prescribes
                         (three dense products, the weight generation per direction, the dC contraction).  The kernels use
                         W = C N associatively and EXECUTE 2.65x fewer flops: executed_tflops and
                         executed_frac_of_mfma_peak (and everything under `roofline`) say how busy the matrix cores really are.
  roofline               the single slowest kernel of the step (bwd_dc_dyc_kernel: t = dy C and the partial sums of dC), timed alone
                         between HIP events on the launch stream: achieved / frac on the flops the kernel EXECUTES against the
                         dense bf16 MFMA peak; `kernels` gives the same for all three kernels of the step, `step.bound_time_us`
                         the least the step could take (executed flops at the MFMA peak, or the bytes it must move at the HBM
                         peak), `backward_call.frac_on_prescribed_flops` the dense-equivalent figure the metric's `value` is
                         made of; traffic is read from profiles/bench_c2_hbm_traffic.md (rocprofv3 FETCH_SIZE / WRITE_SIZE of
                         this script)
  cpu_baseline           the CPU restatement (materialise-then-matmul: oracle C + torch.matmul fp32) on all host cores
  compare, other_configs one-call entry points, kernels that form W on chip, materialise-to-HBM + dense GEMM, dense GEMM;
                         the small-k fp32 layer, the k = 1024 layer, the 12-layer model, the vector-coef (reference) form
"""
import argparse
import ctypes
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X dense fp32 matrix
HBM_PEAK_TBPS = 8.0
T, IN_F, OUT_F, K, SEED = 8192, 768, 3072, 256, 0

F_PER_PRODUCT = 2.0 * T * IN_F * OUT_F + 2.0 * OUT_F * IN_F * K      # one dense product + one W generation / dC contraction
F_STEP = 3.0 * F_PER_PRODUCT
# what the factored kernels execute: z = x N^T, y = z C^T | t = dy C, dx = t N, dC = dy^T z
EXEC_FWD = 2.0 * T * K * (IN_F + OUT_F)
EXEC_BWD = 2.0 * T * K * (OUT_F + IN_F) + 2.0 * T * K * OUT_F
EXEC_STEP = EXEC_FWD + EXEC_BWD
SETTLE_STEPS = 400   # untimed, before the warm-up steps: about 30 ms of continuous work
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_c2_hbm_traffic.md")


def profiled_traffic(kernels):
    """HBM bytes per launch (read + written, scaled by the copy calibration) of the named kernels, summed, from the committed
    counter summary; None when the summary or one of the kernels is missing from it."""
    try:
        rows = [ln for ln in open(TRAFFIC_PROFILE, encoding="utf-8") if ln.startswith("| `rdb::")]
    except OSError:
        return None
    total = 0.0
    for name in kernels:
        hit = [ln for ln in rows if re.match(r"\| `rdb::" + re.escape(name) + r"\b", ln)]
        if not hit:
            return None
        cells = [c.strip() for c in hit[0].strip().strip("|").split("|")]
        total += (float(cells[4]) + float(cells[5])) * 1e6   # columns: kernel, launches, FETCH KiB, WRITE KiB, read MB, written MB
    return total


class LayerBuffers:
    """One set of device buffers of the headline layer and the C-ABI calls of a step on them."""

    def __init__(self, L, _lib, torch, dev, gen, share_inputs_of=None):
        self.L, self._lib = L, _lib
        vp = ctypes.c_void_p
        if share_inputs_of is None:
            self.x = torch.randn(T, IN_F, generator=gen).bfloat16().to(dev)
            self.dy = torch.randn(T, OUT_F, generator=gen).bfloat16().to(dev)
            self.C = (torch.randn(OUT_F, K, generator=gen) * (3 * 0.02**2 / K) ** 0.5).bfloat16().to(dev)
        else:   # other memory, same values
            self.x, self.dy, self.C = (t.clone() for t in (share_inputs_of.x, share_inputs_of.dy, share_inputs_of.C))
        self.y = torch.empty(T, OUT_F, dtype=torch.bfloat16, device=dev)
        self.dx = torch.empty(T, IN_F, dtype=torch.bfloat16, device=dev)
        self.dC = torch.empty(OUT_F, K, dtype=torch.float32, device=dev)
        d = _lib.LinearDesc()
        d.tokens, d.in_f, d.out_f, d.k, d.coef_rows = T, IN_F, OUT_F, K, OUT_F
        d.sO, d.sI, d.seed = IN_F, 1, SEED
        d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_BF16, _lib.RDB_BF16, _lib.RDB_ALGO_AUTO
        self.d, self.dref = d, ctypes.byref(d)
        # caller-owned scratch, sized by the library
        self.ws_bytes = max(L.rdb_linear_workspace_bytes(op, self.dref) for op in (
            _lib.RDB_OP_LINEAR_FWD, _lib.RDB_OP_LINEAR_BWD_DX, _lib.RDB_OP_LINEAR_BWD_DCOEF, _lib.RDB_OP_LINEAR_BWD_PROJECTED))
        self.ws = torch.empty(max(self.ws_bytes, 16), dtype=torch.uint8, device=dev)
        self.state_bytes = L.rdb_linear_projection_bytes(self.dref)
        assert self.state_bytes > 0, "the projected form must apply to the headline workload"
        self.state = torch.empty(self.state_bytes, dtype=torch.uint8, device=dev)
        self.stream = vp(torch.cuda.current_stream().cuda_stream)
        self.p = p = {n: vp(getattr(self, n).data_ptr()) for n in ("x", "dy", "C", "y", "dx", "dC", "ws", "state")}
        # the two calls of a step with their arguments marshalled once: the timed loop is the calls and nothing else
        self._step_calls = (
            (L.rdb_linear_project_fwd, (p["y"], OUT_F, p["state"], p["x"], IN_F, p["C"], None, self.dref, self.stream)),
            (L.rdb_linear_bwd_projected, (p["dx"], IN_F, p["dC"], p["dy"], OUT_F, p["state"], p["C"], self.dref, p["ws"], self.ws_bytes, self.stream)),
        )

    def project(self):
        p = self.p
        self._lib.check(self.L.rdb_linear_project(p["state"], p["x"], IN_F, p["C"], self.dref, self.stream), "rdb_linear_project")

    def project_fwd(self):
        p = self.p
        self._lib.check(self.L.rdb_linear_project_fwd(p["y"], OUT_F, p["state"], p["x"], IN_F, p["C"], None, self.dref, self.stream),
                        "rdb_linear_project_fwd")

    def fwd_projected(self):
        p = self.p
        self._lib.check(self.L.rdb_linear_fwd_projected(p["y"], OUT_F, p["state"], p["C"], None, self.dref, self.stream), "rdb_linear_fwd_projected")

    def bwd(self):
        p = self.p
        self._lib.check(self.L.rdb_linear_bwd_projected(p["dx"], IN_F, p["dC"], p["dy"], OUT_F, p["state"], p["C"], self.dref, p["ws"],
                                                        self.ws_bytes, self.stream), "rdb_linear_bwd_projected")

    def bwd_part(self, part):
        p = self.p
        self._lib.check(self.L.rdb_linear_bwd_projected_part(part, p["dx"], IN_F, p["dC"], p["dy"], OUT_F, p["state"], p["C"], self.dref, p["ws"],
                                                             self.ws_bytes, self.stream), "rdb_linear_bwd_projected_part")

    def dx_separate(self):
        p = self.p
        self._lib.check(self.L.rdb_linear_bwd_dx(p["dx"], IN_F, p["dy"], OUT_F, p["C"], None, self.dref, p["ws"], self.ws_bytes, self.stream),
                        "rdb_linear_bwd_dx")

    def dcoef_separate(self):
        p = self.p
        self._lib.check(self.L.rdb_linear_bwd_dcoef_projected(p["dC"], p["dy"], OUT_F, p["state"], self.dref, self.stream),
                        "rdb_linear_bwd_dcoef_projected")

    def step(self, stream=None):
        """the two calls; `stream` (a ctypes pointer) replaces the stream they were marshalled for (graph capture)"""
        rc = 0
        for fn, a in self._step_calls:
            rc |= fn(*a) if stream is None else fn(*a[:-1], stream)
        if rc:
            self._lib.check(rc, "a call of the step")


def make_event_ms(torch):
    def event_ms(fn, iters):
        """mean duration of fn over `iters` back-to-back calls, HIP events on the launch stream"""
        for _ in range(max(3, min(iters, 50))):
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

    return event_ms


def llm_layer_config(event_ms, torch, L, _lib, dev, g, vendor=True):
    """LLM-sized layer: 4096 -> 14336, k = 1024, 4096 tokens, bf16, forward + backward through the C ABI, every buffer
    allocated beforehand.  The headline of this entry is on the flops the kernels execute."""
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    Tl, in_f, out_f, k = 4096, 4096, 14336, 1024
    x = torch.randn(Tl, in_f, generator=g).bfloat16().to(dev)
    dy = torch.randn(Tl, out_f, generator=g).bfloat16().to(dev)
    C = (torch.randn(out_f, k, generator=g) / 64.0 * (3.0 / k) ** 0.5).bfloat16().to(dev)
    y = torch.empty(Tl, out_f, dtype=torch.bfloat16, device=dev)
    dx = torch.empty(Tl, in_f, dtype=torch.bfloat16, device=dev)
    dC = torch.empty(out_f, k, dtype=torch.float32, device=dev)
    d = _lib.LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = Tl, in_f, out_f, k, out_f, in_f, 1, 0
    d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_BF16, _lib.RDB_BF16, _lib.RDB_ALGO_AUTO
    r = ctypes.byref(d)
    state = torch.empty(L.rdb_linear_projection_bytes(r), dtype=torch.uint8, device=dev)
    wsb = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_PROJECTED, r)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
    px, pdy, pC, py, pdx, pdC, pst, pws = (vp(t.data_ptr()) for t in (x, dy, C, y, dx, dC, state, ws))

    def llm_fwd():
        _lib.check(L.rdb_linear_project(pst, px, in_f, pC, r, stream), "rdb_linear_project")
        _lib.check(L.rdb_linear_fwd_projected(py, out_f, pst, pC, None, r, stream), "rdb_linear_fwd_projected")

    def llm_bwd():
        _lib.check(L.rdb_linear_bwd_projected(pdx, in_f, pdC, pdy, out_f, pst, pC, r, pws, wsb, stream), "rdb_linear_bwd_projected")

    # 50 warm-up and 50 timed calls each (about 25 ms of continuous work per figure: the clocks have settled)
    fwd_ms, bwd_ms = event_ms(llm_fwd, 50), event_ms(llm_bwd, 50)
    proj_ms = event_ms(lambda: L.rdb_linear_project(pst, px, in_f, pC, r, stream), 50)
    ms = fwd_ms + bwd_ms
    F = 6.0 * Tl * in_f * out_f + 6.0 * out_f * in_f * k
    executed = 4.0 * Tl * k * (in_f + out_f) + 2.0 * Tl * k * out_f
    res = {
        "fwd_ms": round(fwd_ms, 4), "bwd_ms": round(bwd_ms, 4), "fwd_bwd_ms": round(ms, 4),
        "calls_ms": {"rdb_linear_project": round(proj_ms, 4), "rdb_linear_fwd_projected": round(fwd_ms - proj_ms, 4),
                     "rdb_linear_bwd_projected": round(bwd_ms, 4)},
        "kernels": "forward product and first backward launch on 256-wide tiles, one persistent block per compute unit",
        "executed_TFLOPs": round(executed / ms / 1e9, 1), "executed_frac_of_mfma_peak": round(executed / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
        "prescribed_gflop": round(F / 1e9, 1), "executed_gflop": round(executed / 1e9, 1),
        "prescribed_TFLOPs_equivalent": round(F / ms / 1e9, 1),
        "note": "all buffers preallocated; the factored form executes 4.1x fewer flops than the prescribed algorithm at this shape, "
                "so only the executed figure is a utilisation"}
    if vendor:
        zz = torch.randn(Tl, k, device=dev).bfloat16()
        res["vendor_gemm_on_the_factored_shapes_ms"] = {
            "y = z.C^T": round(event_ms(lambda: torch.matmul(zz, C.t(), out=y), 50), 4),
            "t = dy.C": round(event_ms(lambda: torch.matmul(dy, C, out=zz), 50), 4),
            "dC = dy^T.z": round(event_ms(lambda: torch.matmul(dy.t(), zz), 50), 4)}
    return res


def f32_layer_config(event_ms, torch, L, _lib, dev, g, compare=True):
    """The headline layer in fp32 (768 -> 3072, k = 256, 8192 tokens) through the projected calls and through the three one-call
    entry points, every buffer allocated beforehand.  The products run on the bf16 matrix cores on exact three-way splits of
    their fp32 operands (six bf16 matrix instructions for an fp32 product, rdb_set_f32_split); beside them the same calls on
    the fp32 matrix instructions.  "executed" flops are the fp32 products the calls perform; the matrix cores execute six
    times as many bf16 flops."""
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    Tl, in_f, out_f, k = T, IN_F, OUT_F, K
    x = torch.randn(Tl, in_f, generator=g).to(dev)
    dy = torch.randn(Tl, out_f, generator=g).to(dev)
    C = (torch.randn(out_f, k, generator=g) * (3 * 0.02**2 / k) ** 0.5).to(dev)
    y = torch.empty(Tl, out_f, device=dev)
    dx = torch.empty(Tl, in_f, device=dev)
    dC = torch.empty(out_f, k, device=dev)
    px, pdy, pC, py, pdx, pdC = (vp(t.data_ptr()) for t in (x, dy, C, y, dx, dC))

    def calls(algo):
        d = _lib.LinearDesc()
        d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = Tl, in_f, out_f, k, out_f, in_f, 1, SEED
        d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_F32, _lib.RDB_F32, algo
        r = ctypes.byref(d)
        n = max(L.rdb_linear_workspace_bytes(op, r) for op in (_lib.RDB_OP_LINEAR_FWD, _lib.RDB_OP_LINEAR_BWD_DX, _lib.RDB_OP_LINEAR_BWD_DCOEF))
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
        pws = vp(ws.data_ptr())
        keep = (d, ws)
        return (lambda: _lib.check(L.rdb_linear_fwd(py, out_f, px, in_f, pC, None, None, r, pws, n, stream), "rdb_linear_fwd"),
                lambda: _lib.check(L.rdb_linear_bwd_dx(pdx, in_f, pdy, out_f, pC, None, r, pws, n, stream), "rdb_linear_bwd_dx"),
                lambda: _lib.check(L.rdb_linear_bwd_dcoef(pdC, None, pdy, out_f, px, in_f, r, pws, n, stream), "rdb_linear_bwd_dcoef"), keep)

    fwd, bdx, bdc, keep = calls(_lib.RDB_ALGO_AUTO)
    t_fwd, t_dx, t_dc = event_ms(fwd, 50), event_ms(bdx, 50), event_ms(bdc, 50)
    proj = 2.0 * Tl * k * in_f   # z = x.N^T or dx = t.N
    prod = 2.0 * Tl * k * out_f  # y = z.C^T, t = dy.C, dC = dy^T.z
    # the way a training step calls the layer: z = x.N^T computed once, kept in the projection state (fp32) for the backward pass
    d = _lib.LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = Tl, in_f, out_f, k, out_f, in_f, 1, SEED
    d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_F32, _lib.RDB_F32, _lib.RDB_ALGO_AUTO
    r = ctypes.byref(d)
    state = torch.empty(L.rdb_linear_projection_bytes(r), dtype=torch.uint8, device=dev)
    wsb = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_PROJECTED, r)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
    pst, pws = vp(state.data_ptr()), vp(ws.data_ptr())
    p_fwd = lambda: _lib.check(L.rdb_linear_project_fwd(py, out_f, pst, px, in_f, pC, None, r, stream), "rdb_linear_project_fwd")
    p_bwd = lambda: _lib.check(L.rdb_linear_bwd_projected(pdx, in_f, pdC, pdy, out_f, pst, pC, r, pws, wsb, stream), "rdb_linear_bwd_projected")
    tp_fwd, tp_bwd = event_ms(p_fwd, 50), event_ms(p_bwd, 50)
    ms = tp_fwd + tp_bwd
    before = L.rdb_set_f32_split(0)   # the same two calls on the fp32 matrix instructions
    tf_fwd, tf_bwd = event_ms(p_fwd, 50), event_ms(p_bwd, 50)
    L.rdb_set_f32_split(before)
    executed = 2 * proj + 3 * prod
    ms_one = t_fwd + t_dx + t_dc
    res = {
        "calls_ms": {"rdb_linear_project_fwd": round(tp_fwd, 4), "rdb_linear_bwd_projected": round(tp_bwd, 4)},
        "fwd_bwd_ms": round(ms, 4), "executed_gflop": round(executed / 1e9, 1), "executed_TFLOPs": round(executed / ms / 1e9, 1),
        "ratio_to_f32_matrix_instruction_peak": round(executed / ms / 1e9 / MFMA_F32_PEAK_TFLOPS, 4),
        "bf16_matrix_instruction_TFLOPs": round(6 * executed / ms / 1e9, 1),
        "bf16_matrix_instruction_frac_of_peak": round(6 * executed / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
        "prescribed_TFLOPs_equivalent": round(F_STEP / ms / 1e9, 1),
        "on_fp32_matrix_instructions_ms": {"rdb_linear_project_fwd": round(tf_fwd, 4), "rdb_linear_bwd_projected": round(tf_bwd, 4),
                                           "fwd_bwd_ms": round(tf_fwd + tf_bwd, 4),
                                           "frac_of_f32_mfma_peak": round(executed / (tf_fwd + tf_bwd) / 1e9 / MFMA_F32_PEAK_TFLOPS, 4)},
        "one_call_entry_points_ms": {"rdb_linear_fwd": round(t_fwd, 4), "rdb_linear_bwd_dx": round(t_dx, 4), "rdb_linear_bwd_dcoef": round(t_dc, 4),
                                     "sum": round(ms_one, 4), "executed_gflop": round(3 * (proj + prod) / 1e9, 1)},
        "kernels": "f32_gemm_kernel for the five products, noise hashed into the operand tiles; operands split into three bf16 parts "
                   "(exact) on their way into LDS, six v_mfma_f32_32x32x16_bf16 per 16 contraction values of a tile pair, fp32 sums",
        "note": "fp32 activations, coefficients and results at fp32 accuracy (parity 1e-5 against the fp64 oracle, as the fp32 matrix "
                "instructions); z = x.N^T is formed once and kept (fp32) in the projection state; the one-call entry points form it twice"}
    del keep
    if compare:
        gf, gdx, gdc, keep = calls(_lib.RDB_ALGO_TILE)
        res["general_kernels_that_form_w_tiles_ms"] = {"fwd": round(event_ms(gf, 5), 4), "dx": round(event_ms(gdx, 5), 4),
                                                        "dcoef": round(event_ms(gdc, 5), 4)}
        del keep
        zz = torch.randn(Tl, k, device=dev)
        res["vendor_gemm_on_the_factored_shapes_ms"] = {
            "y = z.C^T": round(event_ms(lambda: torch.matmul(zz, C.t(), out=y), 20), 4),
            "t = dy.C": round(event_ms(lambda: torch.matmul(dy, C, out=zz), 20), 4),
            "dC = dy^T.z": round(event_ms(lambda: torch.matmul(dy.t(), zz), 20), 4)}
    return res


def smallk_config(event_ms, torch, L, _lib, dev, g):
    """Small-k fp32 regime: 4096 -> 4096, k = 16, forward at batch 1 / 16 / 256.  "effective" = the bytes a stored-W product
    would move (4*(out*in + B*in + B*out)) over the time; the fused kernel itself reads 4*(B*in + out*k) and writes 4*B*out."""
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    in_f = out_f = 4096
    C = (torch.randn(out_f, 16, generator=g) / 64.0).to(dev)
    small = {}
    for B in (1, 16, 256):
        x = torch.randn(B, in_f, generator=g).to(dev)
        y = torch.empty(B, out_f, device=dev)
        d = _lib.LinearDesc()
        d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = B, in_f, out_f, 16, out_f, in_f, 1, 0
        d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_F32, _lib.RDB_F32, _lib.RDB_ALGO_AUTO
        r = ctypes.byref(d)
        n = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, r)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=dev)
        args = (vp(y.data_ptr()), out_f, vp(x.data_ptr()), in_f, vp(C.data_ptr()), None, None, r, vp(ws.data_ptr()), n, stream)
        _lib.check(L.rdb_linear_fwd(*args), "rdb_linear_fwd")
        ms = event_ms(lambda: L.rdb_linear_fwd(*args), 200)
        stored = 4.0 * (out_f * in_f + B * in_f + B * out_f)
        actual = 4.0 * (B * in_f + out_f * 16 + B * out_f)
        small[f"batch_{B}"] = {"fwd_ms": round(ms, 4), "effective_GBps_vs_stored_W": round(stored / ms / 1e6, 1),
                               "actual_HBM_GBps": round(actual / ms / 1e6, 2)}
    return small


def few_token_config(event_ms, torch, L, _lib, dev, g):
    """Few tokens with the headline k: 4096 -> 4096, k = 256, bf16, 1 / 16 / 64 tokens, the three one-call entry points (the
    vector-ALU kernels of the few-token regime), and the same calls forced onto the matrix-core kernels (algo FACTORED)."""
    from randumb_amd import hip

    in_f = out_f = 4096
    k = 256
    C = (torch.randn(out_f, k, generator=g) * 0.01).bfloat16().to(dev)
    res = {}
    for B in (1, 16, 64):
        x = torch.randn(B, in_f, generator=g).bfloat16().to(dev)
        dy = torch.randn(B, out_f, generator=g).bfloat16().to(dev)
        if B == 1:
            for _ in range(300):   # clocks settle
                hip.linear_fwd(x, C, in_f, out_f, in_f, 1, 0)
        row = {}
        for name, algo in (("", _lib.RDB_ALGO_AUTO), ("matrix_core_kernels_", _lib.RDB_ALGO_FACTORED)):
            row[name + "fwd_ms"] = round(event_ms(lambda: hip.linear_fwd(x, C, in_f, out_f, in_f, 1, 0, algo=algo), 100), 4)
            row[name + "dx_ms"] = round(event_ms(lambda: hip.linear_bwd_dx(dy, C, in_f, out_f, in_f, 1, 0, algo=algo), 100), 4)
            row[name + "dcoef_ms"] = round(event_ms(lambda: hip.linear_bwd_dcoef(dy, x, k, out_f, in_f, out_f, in_f, 1, 0, algo=algo), 100), 4)
        res[f"batch_{B}"] = row
    res["note"] = "through the Python wrappers (an allocation of the result and of the workspace per call included)"
    return res


def gpt_step_config(event_ms, torch, dev, g):
    """GPT-2 small with random-backed linears: 12 layers, d = 768, 12 heads, vocab 50304, k = 256, seeds 0..47, bf16, batch
    8 x 1024 random token ids; one training step (forward + backward).  Attention, norms, embedding, head and loss are stock
    PyTorch; the 48 linears run the projected kernels."""
    from randumb_amd.SillyLayers import listgen, stepgen
    from randumb_amd.gpt import RT_GPT, RT_GPTConfig

    torch.manual_seed(0)
    model = RT_GPT(RT_GPTConfig(int_dim_gen=listgen([256] * 48), seed_gen=stepgen(0, 1))).to(torch.bfloat16).to(dev)
    idx = torch.randint(0, 50304, (8, 1024), generator=g).to(dev)
    tgt = torch.randint(0, 50304, (8, 1024), generator=g).to(dev)

    def gpt_step():
        model.zero_grad(set_to_none=True)
        model(idx, tgt).backward()

    ms = event_ms(gpt_step, 5)
    return {"fwd_bwd_ms": round(ms, 2), "tokens_per_s": round(8192 / ms * 1e3, 0),
            "note": "random-backed qkv/proj/fc/mlp-proj; attention, norms, embedding, head and loss are stock PyTorch"}


def other_configs(event_ms, torch, L, _lib, dev):
    """The other configurations, timed for the record (they are parity-test cases, not the metric)."""
    from randumb_amd import hip

    out = {}
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(0)

    out["in4096_out4096_k16_fp32_matrix_coef"] = smallk_config(event_ms, torch, L, _lib, dev, g)
    out["in4096_out4096_k256_bf16_few_tokens"] = few_token_config(event_ms, torch, L, _lib, dev, g)

    out["in4096_out14336_k1024_T4096_bf16"] = llm_layer_config(event_ms, torch, L, _lib, dev, g)
    out["in768_out3072_k256_T8192_fp32"] = f32_layer_config(event_ms, torch, L, _lib, dev, g)

    # ---- the reference's own (vector-coef, 1-D) form at the headline shape: W = Noise . c with ONE coefficient vector of length
    # k needs k hashes per weight element (604 M per regeneration here): the PRNG-bound regime.  Its data flow is the
    # reference's: materialise W to HBM, dense product, dW to HBM, materialize_bwd.  Rates in hashes per second against the
    # vector ALU's budget (256 CUs x 64 lanes x ~2.4 GHz = 39.3 T lane-operations/s, a hash being ~21 of them).
    c1 = (torch.randn(K, generator=g) * (3 * 0.02**2 / K) ** 0.5).to(dev)
    xh = torch.randn(T, IN_F, generator=g).bfloat16().to(dev)
    dyh = torch.randn(T, OUT_F, generator=g).bfloat16().to(dev)
    hashes = float(OUT_F) * IN_F * K

    def mat_fwd():
        return hip.materialize_fwd(c1, (OUT_F, IN_F), (IN_F, 1), SEED, None, False)

    dW = torch.randn(OUT_F, IN_F, device=dev)
    mf_ms = event_ms(mat_fwd, 5)
    mb_ms = event_ms(lambda: hip.materialize_bwd(dW, K, SEED), 5)

    def vec_step():
        W = mat_fwd().to(torch.bfloat16)
        yy = xh @ W.t()
        W2 = mat_fwd().to(torch.bfloat16)
        dxx = dyh @ W2
        dWW = (dyh.t() @ xh).float()
        return yy, dxx, hip.materialize_bwd(dWW, K, SEED)

    vs_ms = event_ms(vec_step, 3)
    # the fused forward in this form: blocks own tiles of W, all compute units share the hashes; 128 tokens timed
    x128 = xh[:128].contiguous()
    fused_ms = event_ms(lambda: hip.linear_fwd(x128, c1, IN_F, OUT_F, IN_F, 1, SEED), 3)
    out["vector_coef_reference_form_768x3072_k256_T8192"] = {
        "materialize_fwd_ms": round(mf_ms, 4), "materialize_fwd_Thash_per_s": round(hashes / mf_ms / 1e9, 3),
        "materialize_bwd_ms": round(mb_ms, 4), "materialize_bwd_Thash_per_s": round(hashes / mb_ms / 1e9, 3),
        "fwd_bwd_step_ms": round(vs_ms, 4), "prescribed_TFLOPs": round(F_STEP / vs_ms / 1e9, 1),
        "fused_linear_fwd_128_tokens_ms": round(fused_ms, 4), "fused_linear_fwd_Thash_per_s": round(hashes / fused_ms / 1e9, 3),
        "valu_budget_T_lane_ops_per_s": 39.3,
        "note": "PRNG-bound: 3 x 604 M hashes per step on the vector ALU; the matrix-coef form of the headline needs 0.2 M per "
                "256-token tile instead"}
    del dW, xh, dyh

    out["gpt2_small_12L_k256_seeds0to47_bf16_8x1024"] = gpt_step_config(event_ms, torch, dev, g)
    return out


def rbias_layer_config(event_ms, torch, L, _lib, dev, main_set):
    # the reference's default layer: W = C.N + s.noise1d (zero coefficients and a fused random bias at initialisation).
    # What SillyLinear runs: the low-rank share through the projected calls of the headline step (z = x.N^T formed once, by
    # the forward pass), the full-rank random-bias share through kernels of its own on top (rdb_linear_rbias_fwd / _bwd,
    # the latter also reducing d s = <dy.R, x>).  Beside it the one-call entry points (z formed by the forward and again
    # by the coefficient gradient) and the older split with dcoef and d s from dW tiles.
    p, ws_bytes, stream = main_set.p, main_set.ws_bytes, main_set.stream
    sb = torch.tensor([0.02], device=dev).bfloat16()
    ds = torch.empty(1, dtype=torch.float32, device=dev)
    psb, pds, r = ctypes.c_void_p(sb.data_ptr()), ctypes.c_void_p(ds.data_ptr()), main_set.dref
    n_ds = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX_DSCALE, r)
    ws_ds = torch.empty(max(n_ds, 16), dtype=torch.uint8, device=dev)
    pws_ds = ctypes.c_void_p(ws_ds.data_ptr())
    n_rb = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_RBIAS_BWD, r)
    ws_rb = torch.empty(max(n_rb, 16), dtype=torch.uint8, device=dev)
    pws_rb = ctypes.c_void_p(ws_rb.data_ptr())

    def fwd_projected():
        main_set.project_fwd()
        _lib.check(L.rdb_linear_rbias_fwd(p["y"], OUT_F, p["x"], IN_F, psb, r, stream), "rdb_linear_rbias_fwd")

    def bwd_projected():
        main_set.bwd()
        _lib.check(L.rdb_linear_rbias_bwd(p["dx"], IN_F, pds, p["dy"], OUT_F, p["x"], IN_F, psb, r, pws_rb, n_rb, stream), "rdb_linear_rbias_bwd")

    fwd = lambda: _lib.check(L.rdb_linear_fwd(p["y"], OUT_F, p["x"], IN_F, p["C"], psb, None, r, p["ws"], ws_bytes, stream), "rdb_linear_fwd")
    dxs = lambda: _lib.check(L.rdb_linear_bwd_dx_dscale(p["dx"], IN_F, pds, p["dy"], OUT_F, p["x"], IN_F, p["C"], psb, r, pws_ds, n_ds, stream),
                             "rdb_linear_bwd_dx_dscale")
    dco = lambda: _lib.check(L.rdb_linear_bwd_dcoef(p["dC"], None, p["dy"], OUT_F, p["x"], IN_F, r, p["ws"], ws_bytes, stream),
                             "rdb_linear_bwd_dcoef")
    dxf = lambda: _lib.check(L.rdb_linear_bwd_dx(p["dx"], IN_F, p["dy"], OUT_F, p["C"], psb, r, p["ws"], ws_bytes, stream), "rdb_linear_bwd_dx")
    dcf = lambda: _lib.check(L.rdb_linear_bwd_dcoef(p["dC"], pds, p["dy"], OUT_F, p["x"], IN_F, r, p["ws"], ws_bytes, stream),
                             "rdb_linear_bwd_dcoef")
    t = {"fwd": round(event_ms(fwd_projected, 100), 4), "bwd_with_dscale": round(event_ms(bwd_projected, 100), 4)}
    t["step"] = round(sum(t.values()), 4)
    o = {"fwd": round(event_ms(fwd, 20), 4), "dx_and_dscale": round(event_ms(dxs, 20), 4), "dcoef": round(event_ms(dco, 20), 4)}
    o["step"] = round(sum(o.values()), 4)
    t["one_call_entry_points"] = o
    t["with_dscale_from_dw_tiles"] = {"dx": round(event_ms(dxf, 20), 4), "dcoef_and_dscale": round(event_ms(dcf, 20), 4)}
    return t


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--no-compare", action="store_true", help="skip the comparison legs and the other configurations")
    ap.add_argument("--no-graph", action="store_true", help="time eager calls only (profiling runs: one kernel record per launch)")
    ap.add_argument("--vector-coef-only", action="store_true",
                    help="run only the vector-coef (reference form) materialise kernels a few times and exit (counter runs)")
    ap.add_argument("--llm-layer-only", action="store_true",
                    help="run only the 4096 -> 14336, k = 1024 layer (projection, forward, backward through the C ABI) and exit "
                         "(profiling runs)")
    ap.add_argument("--f32-layer-only", action="store_true",
                    help="time only the fp32 form of the headline layer (profiling runs)")
    ap.add_argument("--rbias-layer-only", action="store_true",
                    help="run only the headline layer with the fused random bias (projected calls + random-bias share) and exit")
    ap.add_argument("--smallk-only", action="store_true",
                    help="run only the fp32 4096 -> 4096, k = 16 forward at batch 1 / 16 / 256 and exit (profiling runs)")
    ap.add_argument("--few-tokens-only", action="store_true",
                    help="run only the bf16 4096 -> 4096, k = 256 calls at 1 / 16 / 64 tokens and exit (profiling runs)")
    ap.add_argument("--gpt-only", action="store_true",
                    help="run only the GPT-2 small training step with random-backed linears and exit (profiling runs)")
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
    if args.vector_coef_only:
        c1 = (torch.randn(K, generator=g) * (3 * 0.02**2 / K) ** 0.5).to(dev)
        dW = torch.randn(OUT_F, IN_F, generator=g).to(dev)
        for _ in range(5):
            hip.materialize_fwd(c1, (OUT_F, IN_F), (IN_F, 1), SEED, None, False)
            hip.materialize_bwd(dW, K, SEED)
        torch.cuda.synchronize()
        print(json.dumps({"ran": "vector-coef materialize_fwd / materialize_bwd, 768x3072, k=256, 5 times each"}))
        return
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.smallk_only:
        print(json.dumps({"in4096_out4096_k16_fp32_matrix_coef": smallk_config(make_event_ms(torch), torch, L, _lib, dev, g)}))
        return
    if args.few_tokens_only:
        print(json.dumps({"in4096_out4096_k256_bf16_few_tokens": few_token_config(make_event_ms(torch), torch, L, _lib, dev, g)}))
        return
    if args.gpt_only:
        print(json.dumps({"gpt2_small_12L_k256_seeds0to47_bf16_8x1024": gpt_step_config(make_event_ms(torch), torch, dev, g)}))
        return
    if args.f32_layer_only:
        print(json.dumps({"in768_out3072_k256_T8192_fp32": f32_layer_config(make_event_ms(torch), torch, L, _lib, dev, g, compare=False)}))
        return
    if args.llm_layer_only:
        print(json.dumps({"in4096_out14336_k1024_T4096_bf16": llm_layer_config(make_event_ms(torch), torch, L, _lib, dev, g, vendor=False)}))
        return
    main_set = LayerBuffers(L, _lib, torch, dev, g)
    if args.rbias_layer_only:
        for _ in range(SETTLE_STEPS):   # clocks settle
            main_set.step()
        print(json.dumps({"layer_with_fused_random_bias_ms": rbias_layer_config(make_event_ms(torch), torch, L, _lib, dev, main_set)}))
        return
    sets = [main_set] + [LayerBuffers(L, _lib, torch, dev, g, share_inputs_of=main_set) for _ in range(2)]
    set_mb = sum(t.numel() * t.element_size() for t in (main_set.x, main_set.dy, main_set.y, main_set.dx, main_set.dC, main_set.ws,
                                                       main_set.state, main_set.C)) / 1e6
    step = main_set.step

    # ---- the timed region of the contract: W warm-up steps, then exactly K steps between two synchronisations.
    # A step is five short kernel launches; issued one by one from Python the host needs longer per step than the GPU, so
    # the step is recorded once into a HIP graph (the library neither allocates nor uses memset nodes) and each timed step
    # is one replay of it: the same kernels on the same buffers.  The eager loop is timed beside it.
    # The GPU's clocks take some 20 ms of continuous work to settle after an idle period (from idle the first 50 steps run at
    # 120 us each, steps 250 onward at the steady rate), and a training loop keeps the device busy all the time: before the
    # warm-up steps of the contract the step loop runs untimed for SETTLE_STEPS steps.
    def timed(fn):
        for _ in range(SETTLE_STEPS):
            fn()
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    ms_eager = timed(step)
    ms_graph, launch = None, "eager C-ABI calls"
    if not args.no_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                main_set.step(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            torch.cuda.synchronize()
            ref = [t.clone() for t in (main_set.y, main_set.dx, main_set.dC)]
            for t in (main_set.y, main_set.dx, main_set.dC):
                t.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert all(torch.equal(a, b) for a, b in zip(ref, (main_set.y, main_set.dx, main_set.dC))), "graph replay differs from the eager step"
            ms_graph = timed(graph.replay)
        except Exception as e:   # capture not available: the eager loop is the measurement
            print(f"bench.py: HIP graph capture of the step failed ({e}); timing eager calls", file=sys.stderr)
    if ms_graph is not None and ms_graph < ms_eager:
        ms_per_step, launch = ms_graph, "one HIP graph replay per step (the step's three launches captured once)"
    else:
        ms_per_step = ms_eager
    value = F_STEP / (ms_per_step * 1e-3) / 1e12

    # ---- the same loop over three buffer sets in turn: every step starts with cold caches
    for i in range(SETTLE_STEPS + max(3, args.warmup)):
        sets[i % 3].step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        sets[i % 3].step()
    torch.cuda.synchronize()
    ms_rotating = (time.perf_counter() - t0) * 1e3 / args.steps

    event_ms = make_event_ms(torch)

    ms_events_all = event_ms(step, args.steps)
    # spread of single steps, each between its own pair of events (as triton's do_bench reports: median, 20th, 80th percentile)
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    evs[0].record()
    for i in range(args.steps):
        step()
        evs[i + 1].record()
    torch.cuda.synchronize()
    per_step = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps))
    pct = lambda q: per_step[min(len(per_step) - 1, int(q * len(per_step)))]
    step_events = {"all": round(ms_events_all, 5), "p20": round(pct(0.2), 5), "p50": round(pct(0.5), 5), "p80": round(pct(0.8), 5)}

    iters = max(10, min(args.steps, 50))
    calls = {
        "rdb_linear_project_fwd": event_ms(main_set.project_fwd, iters),
        "rdb_linear_project (separate call)": event_ms(main_set.project, iters),
        "rdb_linear_fwd_projected (separate call)": event_ms(main_set.fwd_projected, iters),
        "rdb_linear_bwd_projected": event_ms(main_set.bwd, iters),
        "rdb_linear_bwd_projected, first launch alone": event_ms(lambda: main_set.bwd_part(1), iters),
        "rdb_linear_bwd_projected, second launch alone": event_ms(lambda: main_set.bwd_part(2), iters),
        "rdb_linear_bwd_dx (separate call)": event_ms(main_set.dx_separate, iters),
        "rdb_linear_bwd_dcoef_projected (separate call)": event_ms(main_set.dcoef_separate, iters),
    }
    main_set.bwd()   # leave the outputs of a whole backward pass behind
    # ---- roofline of the dominant kernel.  The step is three launches: factored_zy_kernel (forward call), bwd_dc_dyc_kernel
    # and bwd_tns_red_kernel (backward call); each is timed alone between HIP events on the launch stream, back to back.
    # What a kernel EXECUTES (the factored algorithm's flops) is what its share of the MFMA peak is taken on.
    kernels = {
        "factored_zy_kernel": {"ms": calls["rdb_linear_project_fwd"], "executed_flop": EXEC_FWD,
                               "min_bytes": 2.0 * (T * IN_F + OUT_F * K + T * OUT_F) + 2.0 * 2 * T * K + 2.0 * OUT_F * K,
                               "does": "z = x.N^T into the state, y = z.C^T"},
        "bwd_dc_dyc_kernel": {"ms": calls["rdb_linear_bwd_projected, first launch alone"], "executed_flop": 2 * 2.0 * T * K * OUT_F,
                              "min_bytes": 2.0 * (T * OUT_F + T * K + OUT_F * K + T * K),
                              "does": "t = dy.C and the token ranges' sums of dC = dy^T.z"},
        "bwd_tns_red_kernel": {"ms": calls["rdb_linear_bwd_projected, second launch alone"], "executed_flop": 2.0 * T * K * IN_F,
                               "min_bytes": 2.0 * (T * K + T * IN_F) + 4.0 * OUT_F * K,
                               "does": "dx = t.N and the ordered sum of dC"},
    }
    dom = max(kernels, key=lambda n: kernels[n]["ms"])
    kd = kernels[dom]
    achieved = kd["executed_flop"] / (kd["ms"] * 1e-3) / 1e12
    traffic = profiled_traffic((dom,))
    # the least a step can take on this chip: the flops it executes at the MFMA peak, or the bytes it must move (inputs once,
    # outputs once, the state written and read) at the HBM peak, whichever is longer
    step_min_bytes = 2.0 * (T * IN_F + T * OUT_F) * 2 + 2.0 * 2 * OUT_F * K + 4.0 * OUT_F * K + 2 * (2.0 * 2 * T * K + 2.0 * OUT_F * K)
    bound_mfma_us, bound_hbm_us = EXEC_STEP / (MFMA_BF16_PEAK_TFLOPS * 1e12) * 1e6, step_min_bytes / (HBM_PEAK_TBPS * 1e12) * 1e6
    bwd_ms = calls["rdb_linear_bwd_projected"]
    roofline = {
        "bound": "mfma",
        "kernel": dom, "kernel_does": kd["does"],
        "achieved": round(achieved, 3), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 5),
        "flops_counted": "the flops this kernel executes (factored algorithm)",
        "executed_gflop_per_launch": round(kd["executed_flop"] / 1e9, 3),
        "avg_kernel_ms": round(kd["ms"], 5),
        "timed": f"HIP events on the launch stream around {iters} back-to-back launches of this kernel alone",
        "traffic": traffic, "traffic_source": "profiles/bench_c2_hbm_traffic.md" if traffic is not None else None,
        "hbm_min_bytes_per_launch": kd["min_bytes"],
        "hbm_frac_on_measured_traffic": None if traffic is None else round(traffic / (kd["ms"] * 1e-3) / 1e12 / HBM_PEAK_TBPS, 5),
        "bound_observed": "neither pipe: waits on vector memory and LDS issue (profiles/bench_c2_sq_counters.md)",
        "kernels": {n: {"ms": round(v["ms"], 5), "executed_gflop": round(v["executed_flop"] / 1e9, 3),
                        "executed_tflops": round(v["executed_flop"] / (v["ms"] * 1e-3) / 1e12, 1),
                        "frac": round(v["executed_flop"] / (v["ms"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 5)} for n, v in kernels.items()},
        # the same backward call on the flops the metric prescribes for it (dx and dC: two dense products, a weight generation and
        # the dC contraction): what `value` is made of, not a utilisation of anything
        "backward_call": {"ms": round(bwd_ms, 5), "prescribed_gflop": round(2 * F_PER_PRODUCT / 1e9, 3),
                          "prescribed_tflops": round(2 * F_PER_PRODUCT / (bwd_ms * 1e-3) / 1e12, 1),
                          "frac_on_prescribed_flops": round(2 * F_PER_PRODUCT / (bwd_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 5),
                          "executed_gflop": round(EXEC_BWD / 1e9, 3),
                          "executed_frac": round(EXEC_BWD / (bwd_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 5)},
        "step": {"executed_gflop": round(EXEC_STEP / 1e9, 3), "min_bytes": step_min_bytes,
                 "bound_time_us": round(max(bound_mfma_us, bound_hbm_us), 2), "bound_time_mfma_us": round(bound_mfma_us, 2),
                 "bound_time_hbm_us": round(bound_hbm_us, 2), "measured_us": round(ms_per_step * 1e3, 2),
                 "frac": round(EXEC_STEP / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 5)},
        "calls_ms": {n: round(v, 5) for n, v in calls.items()},
    }

    compare = other = None
    if not args.no_compare:
        x, dy, C = main_set.x, main_set.dy, main_set.C
        d, p, ws_bytes, stream = main_set.d, main_set.p, main_set.ws_bytes, main_set.stream

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
            # the three dense products of the factored algorithm given to the vendor GEMM (torch.matmul)
            zz = torch.randn(T, K, device=dev).bfloat16()
            yy = torch.empty(T, OUT_F, device=dev, dtype=torch.bfloat16)
            tt = torch.empty(T, K, device=dev, dtype=torch.bfloat16)
            cc = torch.empty(OUT_F, K, device=dev, dtype=torch.bfloat16)
            return {"y = z.C^T": round(event_ms(lambda: torch.matmul(zz, C.t(), out=yy), 30), 4),
                    "t = dy.C": round(event_ms(lambda: torch.matmul(dy, C, out=tt), 30), 4),
                    "dC = dy^T.z": round(event_ms(lambda: torch.matmul(dy.t(), zz, out=cc), 30), 4)}

        def onecall_ms(algo):
            dd = _lib.LinearDesc.from_buffer_copy(d)
            dd.algo = algo
            r = ctypes.byref(dd)
            fwd = lambda: _lib.check(L.rdb_linear_fwd(p["y"], OUT_F, p["x"], IN_F, p["C"], None, None, r, p["ws"], ws_bytes, stream), "rdb_linear_fwd")
            dxf = lambda: _lib.check(L.rdb_linear_bwd_dx(p["dx"], IN_F, p["dy"], OUT_F, p["C"], None, r, p["ws"], ws_bytes, stream), "rdb_linear_bwd_dx")
            dcf = lambda: _lib.check(L.rdb_linear_bwd_dcoef(p["dC"], None, p["dy"], OUT_F, p["x"], IN_F, r, p["ws"], ws_bytes, stream),
                                     "rdb_linear_bwd_dcoef")
            return {"fwd": round(event_ms(fwd, 20), 4), "dx": round(event_ms(dxf, 20 if algo != _lib.RDB_ALGO_TILE else 3), 4),
                    "dcoef": round(event_ms(dcf, 20), 4)}

        def strip_ms():
            # the algorithm that does form W, never in HBM: forward strip, dx from a noise strip kept in LDS, dcoef from dW tiles
            t = onecall_ms(_lib.RDB_ALGO_STRIP)
            return {"fwd_strip": t["fwd"], "dx_noise_strip": t["dx"], "dcoef_dw_tile": t["dcoef"],
                    "step": round(t["fwd"] + t["dx"] + t["dcoef"], 4), "dx_tile": onecall_ms(_lib.RDB_ALGO_TILE)["dx"]}

        def python_surface_ms():
            # the same layer through the drop-in surface: SillyLinear (autograd function, ctypes binding), host clock per forward +
            # backward with the GPU kept busy; what a model built from the layer pays per layer when the host is the limit
            from randumb_amd.SillyLayers import SillyLinear

            lin = SillyLinear(IN_F, OUT_F, [K, K], [SEED, SEED + 1], bias=False, device=dev, dtype=torch.bfloat16, matrix_coef=True)
            with torch.no_grad():
                lin.weight_coef.copy_(C)
                lin.weight_scale_bias.zero_()
            xs = x.clone().requires_grad_()

            def layer_step():
                xs.grad = None
                lin.weight_coef.grad = None
                lin(xs).backward(dy)

            for _ in range(100):
                layer_step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(300):
                layer_step()
            torch.cuda.synchronize()
            return round((time.perf_counter() - t0) * 1e3 / 300, 4)

        compare = {
            "one_call_entry_points_ms": onecall_ms(_lib.RDB_ALGO_AUTO),
            "python_surface_SillyLinear_fwd_bwd_wall_ms": python_surface_ms(),
            "layer_with_fused_random_bias_ms": rbias_layer_config(event_ms, torch, L, _lib, dev, main_set),
            "w_tiles_formed_on_chip_ms": strip_ms(),
            "vendor_gemm_on_the_factored_shapes_ms": vendor_skinny(),
            "materialize_then_gemm_ms": round(event_ms(mat_gemm_step, 10), 4),
            "dense_gemm_only_ms": round(event_ms(dense_step, 20), 4),
        }
        del Wd
        other = other_configs(event_ms, torch, L, _lib, dev)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import oracle

        oracle.build()
        ncpu = os.cpu_count() or 1
        torch.set_num_threads(ncpu)
        xc, dyc, Cc = main_set.x.float().cpu(), main_set.dy.float().cpu(), main_set.C.float().cpu().numpy()

        def cpu_step():
            W = torch.from_numpy(oracle.materialize_fwd(Cc, (OUT_F, IN_F), (IN_F, 1), SEED, row_len=IN_F, acc_double=False))
            yy = xc @ W.t()
            W2 = torch.from_numpy(oracle.materialize_fwd(Cc, (OUT_F, IN_F), (IN_F, 1), SEED, row_len=IN_F, acc_double=False))
            dxx = dyc @ W2
            dW = dyc.t() @ xc
            dCC = oracle.materialize_bwd(dW.numpy(), K, SEED, coef_rows=OUT_F)
            return yy, dxx, dCC

        for _ in range(3):
            cpu_step()
        times = []
        for _ in range(10):
            c0 = time.perf_counter()
            cpu_step()
            times.append((time.perf_counter() - c0) * 1e3)
        c_ms = statistics.median(times)
        cpu_baseline = {
            "value": round(F_STEP / (c_ms * 1e-3) / 1e12, 5), "unit": "TFLOP/s", "cores": int(oracle.lib().rdbo_num_threads()),
            "kind": "port", "ms_per_step": round(c_ms, 2), "os_cpu_count": ncpu, "torch_num_threads": int(torch.get_num_threads()),
            "omp_num_threads_env": os.environ.get("OMP_NUM_THREADS"),
            "sample": "median of 10 full fwd+bwd steps of the same workload after 3 warm-ups, fp32: oracle C materialise (OpenMP) + "
                      "torch.matmul",
        }

    out = {
        "metric": "fused PRNG-GEMM fwd+bwd TFLOP/s & % MFMA peak at 768->3072,k=256,8192 tok",
        "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "single fused layer 768->3072, k=256 matrix-coef, 8192 tokens, bf16 act / fp32 accumulate, fwd+dx+dcoef",
                   "tokens": T, "in": IN_F, "out": OUT_F, "k": K, "seed": SEED, "algorithmic_gflop_per_step": round(F_STEP / 1e9, 3),
                   "executed_gflop_per_step": round(EXEC_STEP / 1e9, 3),
                   "algorithm": "factored: y=(x N^T) C^T, dx=(dy C) N, dC=dy^T (x N^T); z = x N^T computed once per step",
                   "value_is": "prescribed-algorithm flops F over the step time (dense-equivalent); the kernels execute "
                               "executed_gflop_per_step", "buffer_set_MB": round(set_mb, 1)},
        "settle_steps": SETTLE_STEPS,
        "frac_of_mfma_peak": round(value / MFMA_BF16_PEAK_TFLOPS, 5),
        "executed_tflops": round(EXEC_STEP / (ms_per_step * 1e-3) / 1e12, 3),
        "executed_frac_of_mfma_peak": round(EXEC_STEP / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 5),
        "ms_per_step_eager": round(ms_eager, 5), "ms_per_step_graph": None if ms_graph is None else round(ms_graph, 5), "launch": launch,
        "ms_per_step_rotating": round(ms_rotating, 5),
        "value_rotating": round(F_STEP / (ms_rotating * 1e-3) / 1e12, 3),
        "ms_per_step_events": step_events,
        "roofline": roofline, "cpu_baseline": cpu_baseline, "compare": compare, "other_configs": other,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
