"""Benchmark of the quantized Mamba1 mixer prefill hot path on one MI355X.

One step = one pass of the path over one batch of synthetic input, at the Mamba1-2.8b prefill
shape (batch 8, seqlen 2048, d_model 2560, d_inner 5120, d_state 16, conv width 4):

    in_proj   W8A8 GEMM  [2560 -> 10240], int8 out, seqlen-last layout  (x | z halves)
    conv1d    int8 depthwise causal conv + SiLU + requant on the x half
    sscan     int8 selective scan with z gating, fp16 out (batch, seqlen, d_inner), fp32 last state
    out_proj  W8A8 GEMM  [5120 -> 2560], fp16 out

Inputs are resident in HBM before the timed region.  dt, B and C (produced by x_proj / dt_proj in
the full layer) and out_proj's int8 input (produced by the Hadamard-quantise op) are synthetic
tensors of the right shape and layout.  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from quamba_amd import QCausalConv1D, W8A8B8O8Linear, W8A8B16O16Linear, ops, synth  # noqa: E402

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA
F16_PEAK_TFLOPS = 2500.0    # MI355X dense fp16 MFMA

CFG = dict(batch=8, seqlen=2048, d_model=2560, d_inner=5120, d_state=16, dt_rank=160, d_conv=4)


def _t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _s(v, dev):
    return torch.tensor([float(v)], dtype=torch.float32, device=dev)


class Mixer:
    """Holds the resident tensors of one mixer and runs the four kernels in order."""

    def __init__(self, dev, batch, seqlen, cfg=CFG, seed=1234, input_sets=1):
        self.dev = dev
        B, L = batch, seqlen
        D, dm, N, k = cfg["d_inner"], cfg["d_model"], cfg["d_state"], cfg["d_conv"]
        self.B, self.L, self.D, self.dm, self.N = B, L, D, dm, N
        g = synth.rng_for(seed, "hidden")
        # hidden states after the (out-of-scope) int8 RMSNorm: outlier channels, per-tensor scale
        hid = synth.activations((B * L, dm), 1, seed, "hidden")
        q_hid, s_hid = synth.quantize_absmax(hid)
        self.hidden = _t(q_hid, dev).view(B, L, dm)

        # int8 weights with one scale per output channel (the [1, N] b_scales epilogue of the reference's
        # W8A8B8O8LinearParallel, quamba/qLinearLayer.py:698-711)
        w_in_q, w_in_s, _ = synth.linear_weights(2 * D, dm, seed, "in_proj", per_channel=True)
        self.in_proj = W8A8B8O8Linear(dm, 2 * D, device=dev)
        self.in_proj.weight = _t(w_in_q, dev).t()
        s_xz = 0.04                                          # int8 scale of in_proj's output
        self.in_proj.a = torch.tensor([[float(s_hid) / s_xz]], dtype=torch.float32, device=dev)
        self.in_proj.b = _t(w_in_s, dev).view(1, 2 * D)

        qw, sw, qb, sb = synth.conv_weights(D, k, seed)
        self.conv = QCausalConv1D(D, D, k, groups=D, device=dev)
        self.conv.weight, self.conv.bias = _t(qw, dev), _t(qb, dev)
        self.conv.weight_scale, self.conv.bias_scale = float(sw), float(sb)
        self.conv.input_scale, self.conv.output_scale = s_xz, 0.03

        sc = synth.mamba1_scan_inputs(1, 8, D, N, seed=seed)    # parameters only (A_log, D, dt_bias + scales)
        self.A_log, self.Dq, self.dt_bias = _t(sc["A_log"], dev), _t(sc["D"], dev), _t(sc["dt_bias"], dev)
        self.s_A, self.s_D, self.s_db = _s(sc["s_A"], dev), _s(sc["s_D"], dev), _s(sc["s_db"], dev)
        self.s_u, self.s_z = _s(self.conv.output_scale, dev), _s(s_xz, dev)
        # dt as dt_proj.to_seqlen_last leaves it: (B, D, L) view of a [D][B][L] buffer
        dt_target = np.exp(g.uniform(np.log(1e-3), np.log(1e-1), (D, B, L))).astype(np.float32)
        dt_bias_f = sc["dt_bias"].astype(np.float32) * sc["s_db"]
        dt_raw = synth.inv_softplus(dt_target.astype(np.float64)) - dt_bias_f[:, None, None]
        q_dt, s_dt = synth.quantize_absmax(dt_raw.astype(np.float32))
        self.dt = _t(q_dt, dev).transpose(0, 1)
        self.s_dt = _s(s_dt, dev)
        qB, sB = synth.quantize_absmax(synth.activations((B, 1, N, L), 2, seed, "B", outliers=False))
        qC, sC = synth.quantize_absmax(synth.activations((B, 1, N, L), 2, seed, "C", outliers=False))
        self.Bm, self.Cm, self.s_B, self.s_C = _t(qB, dev), _t(qC, dev), _s(sB, dev), _s(sC, dev)
        self.s_state = _s(1.0, dev)

        w_out_q, w_out_s, _ = synth.linear_weights(dm, D, seed, "out_proj", per_channel=True)
        self.out_proj = W8A8B16O16Linear(D, dm, device=dev)
        self.out_proj.weight = _t(w_out_q, dev).t()
        self.out_proj.a = torch.tensor([[0.02]], dtype=torch.float32, device=dev)
        self.out_proj.b = _t(w_out_s, dev).view(1, dm)
        y_q, _ = synth.quantize_absmax(synth.activations((B * L, D), 1, seed, "y_had"))
        self.y_q = _t(y_q, dev).view(B, L, D)
        # Step i reads input set i % input_sets: the first set is the one above, the others hold the same values rolled
        # along the token axis (same distribution, other addresses), so that a step does not find the inputs of the
        # step before in the 256 MB last-level cache.
        self.sets = [(self.hidden, self.dt, self.Bm, self.Cm, self.y_q)]
        for r in range(1, input_sets):
            sh = 97 * r
            self.sets.append((torch.roll(self.hidden, sh, 1).contiguous(),
                              torch.roll(self.dt.transpose(0, 1), sh, 2).contiguous().transpose(0, 1),
                              torch.roll(self.Bm, sh, 3).contiguous(), torch.roll(self.Cm, sh, 3).contiguous(),
                              torch.roll(self.y_q, sh, 1).contiguous()))
        self.calls = 0

    def step(self, events=None, only=None):
        """One pass of the four kernels; events[i] (i = 0..4) is recorded before kernel i / after kernel i - 1,
        all of them or just the positions in `only`."""
        rec = (lambda i: events[i].record() if only is None or i in only else None) if events is not None else (lambda i: None)
        hidden, dt, Bm, Cm, y_q = self.sets[self.calls % len(self.sets)]
        self.calls += 1
        rec(0)
        xz = self.in_proj.to_seqlen_last(hidden)                   # (B, 2D, L), strides (L, B*L, 1)
        rec(1)
        x, z = xz[:, :self.D], xz[:, self.D:]
        xc = self.conv(x)
        rec(2)
        y, state = ops.sscan_fwd(xc, self.s_u, dt, self.s_dt, self.A_log, self.s_A, Bm, self.s_B,
                                 Cm, self.s_C, self.s_state, self.Dq, self.s_D, z, self.s_z, self.dt_bias,
                                 self.s_db, True, state_dtype=torch.float32)
        rec(3)
        out = self.out_proj(y_q)
        rec(4)
        return xz, xc, y, state, out


def kernel_table(B, L, cfg=CFG):
    """Algorithmic (compulsory) bytes and ops of one launch of each kernel."""
    D, dm, N, k = cfg["d_inner"], cfg["d_model"], cfg["d_state"], cfg["d_conv"]
    M = B * L
    return [
        dict(name="in_proj_w8a8_gemm", bound="mfma", ops=2.0 * M * dm * 2 * D, bytes=M * dm + dm * 2 * D + M * 2 * D),
        dict(name="causal_conv1d_fwd", bound="hbm", bytes=2.0 * B * D * L + D * (k + 1)),
        dict(name="sscan_fwd", bound="hbm", bytes=3.0 * B * D * L + 2 * B * N * L + 2 * B * D * L + 4 * B * D * N + D * (N + 2)),
        dict(name="out_proj_w8a8_gemm", bound="mfma", ops=2.0 * M * D * dm, bytes=M * D + D * dm + 2 * M * dm),
    ]


def cpu_baseline(dev_mixer, seconds_budget=30.0):
    """Times the CPU oracle (conv, scan: C restatement with OpenMP) and an fp32 torch.matmul on the
    dequantised GEMM operands, on a batch-1 slice of the same workload, on the host's cores."""
    import oracle
    m = dev_mixer
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    torch.set_num_threads(threads)
    L, D, dm, N = m.L, m.D, m.dm, m.N
    hid = m.hidden[:1].cpu().float().view(L, dm)
    w_in = m.in_proj.weight.t().cpu().float()
    y_q = m.y_q[:1].cpu().float().view(L, D)
    w_out = m.out_proj.weight.t().cpu().float()
    # the conv and the scan take what in_proj produced for this batch entry (x | z halves), as on the GPU
    m.calls = 0                                       # input set 0: the tensors sliced above
    xz = m.step()[0][:1].cpu().numpy()
    x8, z8 = np.ascontiguousarray(xz[:, :D]), np.ascontiguousarray(xz[:, D:])
    dt8 = np.ascontiguousarray(m.dt[:1].cpu().numpy())
    B8, C8 = m.Bm[:1].cpu().numpy(), m.Cm[:1].cpu().numpy()
    A, Dq, db = m.A_log.cpu().numpy(), m.Dq.cpu().numpy(), m.dt_bias.cpu().numpy()
    qw, qb = m.conv.weight.cpu().numpy(), m.conv.bias.cpu().numpy()
    sc = lambda t: float(t.item())

    def one_pass():
        (hid @ w_in.t())
        xc = oracle.conv1d_fwd(x8, qw, qb, m.conv.input_scale, m.conv.weight_scale, m.conv.bias_scale,
                               m.conv.output_scale)
        oracle.sscan_fwd(xc, dt8, A, B8, C8, Dq, db, z8, s_u=sc(m.s_u), s_delta=sc(m.s_dt), s_A=sc(m.s_A),
                         s_B=sc(m.s_B), s_C=sc(m.s_C), s_D=sc(m.s_D), s_db=sc(m.s_db), s_z=sc(m.s_z))
        (y_q @ w_out.t())

    one_pass()                                        # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        one_pass()
        reps += 1
        el = time.perf_counter() - t0
        if (reps >= 3 and el > 0.4 * seconds_budget) or el > seconds_budget:      # about 12 s of CPU work
            break
    per_pass = (time.perf_counter() - t0) / reps
    return dict(value=L / per_pass, unit="tokens/s", cores=threads, kind="port",
                sample=f"batch 1 of {m.B} (seqlen {L}, same weights and shapes), {reps} passes after 1 warm-up; "
                       "conv and scan: C oracle with OpenMP; GEMMs: fp32 torch.matmul on dequantised operands")


SETTLE_MS = 40.0     # untimed repetitions before a measurement (main sets it from --settle-ms)


def _time_fn(fn, steps, warmup, settle_ms=None):
    """Mean time of `steps` calls in ms (HIP events around the whole run), after `warmup` calls and, before them, as many
    untimed calls as fill `settle_ms`, queued without host synchronisation: the part takes about 30 ms of a new
    workload to settle its clocks, and an idle gap lets them fall again."""
    settle_ms = SETTLE_MS if settle_ms is None else settle_ms
    if settle_ms > 0:
        fn()                                # (the first call may allocate or load code: not a measure of the others)
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        est_ms = max((time.perf_counter() - t) * 1e3, 0.02)
        for _ in range(int(min(2000, settle_ms / est_ms))):
            fn()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def _ri(dev):
    return lambda *s: torch.randint(-128, 128, s, dtype=torch.int8, device=dev)


def _wl_decode(dev):
    """Mamba1-2.8b decode step at batch 64, fp32 state, sixteen steps in one HIP graph.  The row's headline figures
    (`us`, `tokens_per_s`, `frac`) are the two launches the layer executes - conv update, then state update, with
    x_proj / dt_proj between them in the full layer - on the benchmark configuration's int8 conv state [64, 5120, 3].
    `us_one_launch` is the fused kernel (dt, B and C given beforehand), `state_width_4` the same pair of figures on the
    (B, D, d_conv) buffer the reference's mixer allocates."""
    ri = _ri(dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    B, D, N = 64, 5120, 16
    conv = QCausalConv1D(D, D, 4, groups=D, device=dev)
    conv.weight, conv.bias = ri(D, 4), ri(D)
    conv.weight_scale, conv.bias_scale, conv.input_scale, conv.output_scale = 0.004, 0.004, 0.04, 0.03
    ssm_state = torch.randn(B, D, N, device=dev) * 0.1
    ring = [(ri(B, D), ri(B, D), ri(B, N), ri(B, N), ri(B, D)) for _ in range(16)]
    A, Dq, db = ri(D, N), ri(D), ri(D)
    it = [0]
    s_x, s_dt, s_A, s_B, s_C, s_D, s_z, s_db = (sc(v) for v in (0.03, 0.02, 0.02, 0.03, 0.03, 0.008, 0.04, 0.01))

    # the same 16 steps captured into one HIP graph (how decode loops are run in practice)
    def graphed(step):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(16):
                step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(16):
                step()
        return _time_fn(graph.replay, 64, 4) / 16

    def measure(width):
        conv_state = ri(B, D, width)

        def decode():
            x, dt, Bv, Cv, z = ring[it[0] % 16]
            it[0] += 1
            xc = conv.update(x, conv_state)
            ops.sscan_update(ssm_state, xc, s_x, dt, s_dt, A, s_A, None, Bv, s_B, Cv, s_C, Dq, s_D, z, s_z, db, s_db, True)

        def decode_one_launch():
            x, dt, Bv, Cv, z = ring[it[0] % 16]
            it[0] += 1
            ops.mamba1_decode_step(x, conv_state, conv.input_scale, conv.weight, conv.weight_scale, conv.output_scale,
                                   conv.bias_scale, conv.bias, True, ssm_state, dt, s_dt, A, s_A, None, Bv, s_B, Cv, s_C, Dq,
                                   s_D, z, s_z, db, s_db, True, x_scale=s_x)
        ms_eager = _time_fn(decode, 208, 16)
        return graphed(decode), graphed(decode_one_launch), ms_eager

    ms_two, ms_one, ms_eager = measure(3)
    ms_two4, ms_one4, _ = measure(4)
    nbytes = 3 * B * D + 2 * B * D * 3 + 2 * B * D * N * 4 + 2 * B * D + D * N
    return dict(workload="Mamba1-2.8b decode step (conv update, then state update: two launches), batch 64, fp32 state, "
                         "int8 conv state [64,5120,3], HIP graph of 16 steps",
                name="decode_step", us=ms_two * 1e3, us_one_launch=ms_one * 1e3, us_eager_python=ms_eager * 1e3,
                state_width_4=dict(us=ms_two4 * 1e3, us_one_launch=ms_one4 * 1e3),
                tokens_per_s=B / ms_two * 1e3, bound="hbm", bytes=nbytes, achieved_GBs=nbytes / ms_two / 1e6,
                frac=nbytes / ms_two / 1e6 / HBM_PEAK_GBS,
                one_launch=dict(tokens_per_s=B / ms_one * 1e3, achieved_GBs=nbytes / ms_one / 1e6,
                                frac=nbytes / ms_one / 1e6 / HBM_PEAK_GBS))


def _wl_ssd(dev, steps, warmup, B, L, H, N, G, Q, name, label, fp32_dt=False):
    """SSD chunk scan of `label`: x scales per (ssd group, four head groups, four dim groups), B and C scales per ssd
    group; step sizes as int8 codes with bias and softplus in the kernel, or (`fp32_dt`) already processed, fp32 in
    [1e-3, 1e-1]; fp32 final states."""
    ri = _ri(dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    x, Bm, Cm = ri(B, L, H, 64), ri(B, L, G, N), ri(B, L, G, N)
    if fp32_dt:
        dt = torch.exp(torch.rand(B, L, H, device=dev) * (np.log(1e-1) - np.log(1e-3)) + np.log(1e-3)).float()
    else:
        dt = ri(B, L, H)
    A2, D2 = ri(H), ri(H)
    bias = torch.zeros(H, dtype=torch.float16, device=dev)
    # scales live on the device before the timed region (creating one is a blocking host-to-device copy)
    k_dt, k_A, k_D = (sc(v) for v in (0.02, 0.02, 0.008))
    hpg = H // G
    k_x = torch.rand(G, 4, 4, device=dev) * 0.02 + 0.02
    k_B, k_C = torch.rand(G, device=dev) * 0.02 + 0.02, torch.rand(G, device=dev) * 0.02 + 0.02
    kw = dict(x_head_group_range=(torch.arange(1, 5, dtype=torch.int32, device=dev) * (hpg // 4)).repeat(G, 1),
              x_dim_group_range=(torch.arange(1, 5, dtype=torch.int32, device=dev) * 16).repeat(G, 4, 1))
    ssd = lambda: ops.ssd_chunk_scan_combined_fwd(x, k_x, dt, k_dt, A2, k_A, Bm, k_B, Cm, k_C, None, Q,
                                                  q_D=D2, D_scale=k_D, dt_bias=bias, dt_softplus=True,
                                                  final_state_dtype=torch.float32, **kw)
    ms = _time_fn(ssd, steps, warmup)
    # the same call captured into a HIP graph (how a serving loop would issue it): without the eager launches' work at
    # every kernel boundary
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ssd()
    ms_graph = _time_fn(graph.replay, steps, warmup)
    del graph
    nbytes = B * L * H * 64 + 2 * B * L * G * N + B * L * H * (4 if fp32_dt else 1) + 2 * B * L * H * 64 + 4 * B * H * 64 * N
    # dense multiply-adds: C B^T (lower tiles), chunk states, C x entering state, causal part of (C B^T) x
    nc = (L + Q - 1) // Q
    flops = 2.0 * B * nc * (G * Q * Q * N / 2 + H * Q * 64 * N + H * Q * 64 * N + H * Q * Q * 64 / 2)
    # fp16 products (chunk states, C x entering state, causal part of (C B^T) x) against the fp16 matrix peak, and the
    # int8 product C B^T as the kernel forms it - per head, at and below the diagonal in 16 x 32 blocks - against the int8 peak
    f16_flops = 2.0 * B * nc * H * (2 * Q * 64 * N + Q * Q * 64 / 2)
    i8_ops = 2.0 * B * nc * H * N * sum(16 * 32 * ((mt + 2) // 2) for mt in range(Q // 16))
    return dict(workload=label, name=name, us=ms * 1e3, us_hip_graph=ms_graph * 1e3, tokens_per_s=B * L / ms * 1e3, bound="hbm", bytes=nbytes,
                achieved_GBs=nbytes / ms / 1e6, frac=nbytes / ms / 1e6 / HBM_PEAK_GBS, dense_TFLOPs=flops / ms / 1e9,
                mfma_f16_frac=f16_flops / ms / 1e9 / F16_PEAK_TFLOPS, mfma_i8_frac=i8_ops / ms / 1e9 / INT8_PEAK_TOPS)


def _wl_ssd_other_shape(dev, steps, warmup, B, L, H, P, N, Q, label):
    """SSD chunk scan at a shape outside the released models' (other head dimension, state count or chunk length), one
    group, per-tensor scales, fp32 final states: per-launch time and algorithmic bytes."""
    ri = _ri(dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    x, dt, Bm, Cm, A2, D2 = ri(B, L, H, P), ri(B, L, H), ri(B, L, 1, N), ri(B, L, 1, N), ri(H), ri(H)
    bias = torch.zeros(H, dtype=torch.float16, device=dev)
    k_x, k_dt, k_A, k_B, k_C, k_D = (sc(v) for v in (0.03, 0.02, 0.02, 0.03, 0.03, 0.008))
    ssd = lambda: ops.ssd_chunk_scan_combined_fwd(x, k_x, dt, k_dt, A2, k_A, Bm, k_B, Cm, k_C, None, Q, q_D=D2, D_scale=k_D,
                                                  dt_bias=bias, dt_softplus=True, final_state_dtype=torch.float32)
    ms = _time_fn(ssd, steps, warmup)
    nbytes = B * L * H * P + 2 * B * L * N + B * L * H + 2 * B * L * H * P + 4 * B * H * P * N
    return dict(workload=label, us=ms * 1e3, tokens_per_s=B * L / ms * 1e3, bound="hbm", bytes=nbytes,
                achieved_GBs=nbytes / ms / 1e6, frac=nbytes / ms / 1e6 / HBM_PEAK_GBS)


def _wl_w4a8(dev, steps, warmup, M, Nn, K, o8, name):
    ri = _ri(dev)
    a = ri(M, K)
    w = torch.randint(0, 256, (Nn, K // 2), dtype=torch.uint8, device=dev)
    sg = (torch.rand(K // 128, Nn, device=dev) * 10 + 2).half()
    s_ch, s_tok = torch.full((1, Nn), 1e-4, device=dev), torch.ones(M, device=dev)
    fn = ops.w4a8o8_gemm if o8 else ops.w4a8o16_gemm
    ms = _time_fn(lambda: fn(a, w, s_tok, s_ch, sg, None, M, Nn, K, False), steps, warmup)
    n_ops = 2.0 * M * Nn * K
    tops = n_ops / ms / 1e9
    return dict(workload=f"Mamba2-8b W4A8 {name} {M}x{K}->{Nn}", name=f"w4a8_{name}", us=ms * 1e3, tokens_per_s=M / ms * 1e3,
                bound="mfma", ops=n_ops, achieved_TOPs=tops, frac=tops / INT8_PEAK_TOPS)


SSD_27B = (4, 4096, 80, 128, 1, 256, "ssd_2p7b", "Mamba2-2.7b SSD chunk scan, batch 4 x 4096, 80 heads, d_state 128, chunk 256, "
           "x scales per head group, fp32 step sizes", True)
SSD_8B = (16, 1024, 128, 128, 8, 256, "ssd_8b", "Mamba2-8b SSD chunk scan, batch 16 x 1024, 128 heads, d_state 128, 8 groups, chunk 256")


def secondary_workloads(dev, steps, warmup):
    """The other benchmark configurations on the same path, in short form for the default line: the Mamba1-2.8b decode
    step, the Mamba2-2.7b SSD chunk scan, and the Mamba2-8b layer's three heavy kernels (W4A8 in_proj, SSD chunk scan,
    W4A8 out_proj).  Per-launch time, algorithmic bytes or operations, fraction of the bounding peak."""
    out = [_wl_decode(dev), _wl_ssd(dev, steps, warmup, *SSD_27B),
           _wl_w4a8(dev, steps, warmup, 16384, 18560, 4096, True, "in_proj"),
           _wl_ssd(dev, steps, warmup, *SSD_8B),
           _wl_w4a8(dev, steps, warmup, 16384, 4096, 8192, False, "out_proj")]
    torch.cuda.empty_cache()
    return out


def other_workloads(dev, steps, warmup):
    """Secondary shapes of the same path, the long list: whole mixers for one token and over a prompt, the Mamba2 conv,
    Hadamard and norm kernels, single-token W4A8 streams.  Returns a list of dicts with per-launch time and roofline
    fraction."""
    from quamba_amd import Quamb2Conv1D
    out = []
    ri = _ri(dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    D, N = 5120, 16
    # the whole Mamba1-2.8b mixer for one token (in_proj, conv update, x_proj, dt_proj, state update, Hadamard,
    # out_proj): eight layers with their own weights (330 MB, more than the last-level cache holds) in one graph
    from quamba_amd import W8A8QMamba
    layers = []
    for _ in range(8):
        m = W8A8QMamba(2560, 16, 4, device=dev, state_dtype=torch.float32)
        for name in ("in_proj", "x_proj", "dt_proj", "out_proj"):
            lin = getattr(m, name)
            lin._set_weight(ri(lin.out_features, lin.in_features))
            lin.a, lin.b, lin.alpha = sc(0.5).view(1, 1), sc(1e-3).view(1, 1), 5e-4
        m.conv1d.weight, m.conv1d.bias = ri(D, 4), ri(D)
        m.conv1d.input_scale = m.conv1d.weight_scale = m.conv1d.bias_scale = 0.01
        m.conv1d.output_scale = 0.02
        m.selective_scan.A_log, m.selective_scan.D, m.selective_scan.dt_bias = ri(D, N), ri(D), ri(D)
        m.had.x_H_scale = 0.05
        layers.append(m)
    w_bytes = sum(getattr(layers[0], n).weight.numel() for n in ("in_proj", "x_proj", "dt_proj", "out_proj"))
    for B in (1, 64):
        states = [m.allocate_inference_cache(B) for m in layers]
        h = ri(B, 1, 2560)

        def token():
            for m, (cs, ss) in zip(layers, states):
                m.step(h, cs, ss)
        for _ in range(3):
            token()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            token()
        ms = _time_fn(graph.replay, 64, 4) / len(layers)
        nbytes = w_bytes + B * (2 * D * N * 4 + 2 * D * 3 + 2560 + 2 * 2560)
        out.append(dict(workload=f"Mamba1-2.8b W8A8 mixer, one token (all seven kernels), batch {B}, HIP graph over 8 layers",
                        us=ms * 1e3, tokens_per_s=B / ms * 1e3, bound="hbm", achieved_GBs=nbytes / ms / 1e6,
                        frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
        del graph, states
    # the same mixer module over a whole prompt: W8A8QMamba.forward, batch 8 x 2048 (in_proj, conv writing both
    # layouts, x_proj, dt_proj, selective scan, Hadamard, out_proj, and the small layout copies between them)
    m = layers[0]
    Bp, Lp = 8, 2048
    hp = ri(Bp, Lp, 2560)
    ms = _time_fn(lambda: m.forward(hp), min(steps, 10), 3)
    out.append(dict(workload="Mamba1-2.8b W8A8 mixer forward over a prompt (all seven kernels), batch 8 x 2048",
                    us=ms * 1e3, tokens_per_s=Bp * Lp / ms * 1e3, bound="mfma",
                    achieved_TOPs=2.0 * Bp * Lp * (2560 * 10240 + 5120 * 192 + 160 * 5120 + 5120 * 2560) / ms / 1e9,
                    frac=2.0 * Bp * Lp * (2560 * 10240 + 5120 * 192 + 160 * 5120 + 5120 * 2560) / ms / 1e9 / INT8_PEAK_TOPS))
    del layers, m, hp
    # Mamba2-8b xBC conv: batch 16 x 1024, x 8192 channels (128 heads of 64), 8 groups of d_state 128, grouped scales
    B, L, H, N, G = 16, 1024, 128, 128, 8
    dim = H * 64 + 2 * G * N
    conv2 = Quamb2Conv1D(H * 64, 64, N, G, 4, 4, dim, dim, 4, groups=dim, device=dev)
    conv2.weight, conv2.bias = ri(dim, 4), ri(dim)
    conv2.x_scale = conv2.B_scale = conv2.C_scale = 0.04
    conv2.wx_scale = conv2.wB_scale = conv2.wC_scale = 0.004
    conv2.bx_scale = conv2.bB_scale = conv2.bC_scale = 0.004
    conv2.x_out_scales = torch.rand(G, 4, 4, device=dev) * 0.02 + 0.02
    conv2.B_out_scales, conv2.C_out_scales = torch.rand(G, device=dev) * 0.02 + 0.02, torch.rand(G, device=dev) * 0.02 + 0.02
    conv2.x_head_group_range = torch.tensor([[4, 8, 12, 16]] * G, dtype=torch.int32, device=dev)
    conv2.x_dim_group_range = torch.tensor([[[16, 32, 48, 64]] * 4] * G, dtype=torch.int32, device=dev)
    xBC = ri(B, L, dim).transpose(1, 2)
    ms = _time_fn(lambda: conv2(xBC), steps, warmup)
    nbytes = 2 * B * L * dim + 5 * dim
    out.append(dict(workload="Mamba2-8b xBC conv, batch 16 x 1024, 10240 channels, grouped output scales", us=ms * 1e3,
                    tokens_per_s=B * L / ms * 1e3, bound="hbm", achieved_GBs=nbytes / ms / 1e6,
                    frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
    del xBC
    # the SSD chunk scan at shapes outside the released models': heads of 128 channels (the matrix-core kernels, a head
    # as two heads of 64) and 256 states (the general kernels), both with the 2.7b shape's token and channel counts
    out.append(_wl_ssd_other_shape(dev, min(steps, 10), 2, 4, 4096, 40, 128, 128, 256,
                                   "SSD chunk scan with heads of 128 channels, batch 4 x 4096, 40 heads, d_state 128, chunk 256"))
    out.append(_wl_ssd_other_shape(dev, min(steps, 10), 2, 4, 4096, 80, 64, 256, 256,
                                   "SSD chunk scan with 256 states (general kernels), batch 4 x 4096, 80 heads of 64, chunk 256"))
    torch.cuda.empty_cache()
    # Hadamard + quantisation of the scan output in front of out_proj: 16384 rows of 5120 (40 x 128) and of 8192
    for dim in (5120, 8192):
        xh = torch.randn(16384, dim, device=dev, dtype=torch.float16)
        ms = _time_fn(lambda: ops.hadamard_quant(xh, 0.2), steps, warmup)
        nbytes = 3 * 16384 * dim
        out.append(dict(workload=f"Hadamard + int8 quantisation, 16384 rows x {dim}", us=ms * 1e3, tokens_per_s=16384 / ms * 1e3,
                        bound="hbm", achieved_GBs=nbytes / ms / 1e6, frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
        del xh
    # W4A8 layers for one token: a stream over the packed weights (eight copies in turn: 300 MB)
    for (M, Nn, K, o8, name) in ((16384, 18560, 4096, True, "in_proj"), (16384, 4096, 8192, False, "out_proj")):
        sg = (torch.rand(K // 128, Nn, device=dev) * 10 + 2).half()
        s_ch = torch.full((1, Nn), 1e-4, device=dev)
        fn = ops.w4a8o8_gemm if o8 else ops.w4a8o16_gemm
        ws = [torch.randint(0, 256, (Nn, K // 2), dtype=torch.uint8, device=dev) for _ in range(8)]
        a1, s_tok1 = ri(1, K), torch.ones(1, device=dev)
        for w in ws:
            fn(a1, w, s_tok1, s_ch, sg, None, 1, Nn, K, False)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for w in ws:
                fn(a1, w, s_tok1, s_ch, sg, None, 1, Nn, K, False)
        ms = _time_fn(graph.replay, 64, 4) / len(ws)
        nbytes = Nn * K // 2 + Nn * (K // 128) * 2
        out.append(dict(workload=f"Mamba2-8b W4A8 {name} for one token, 1x{K}->{Nn}, HIP graph", us=ms * 1e3,
                        tokens_per_s=1 / ms * 1e3, bound="hbm", achieved_GBs=nbytes / ms / 1e6,
                        frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
        del graph, ws
    # gated RMS norm of the Mamba2-8b mixer: 16384 rows x 8192, fp16 in, int8 gate, fp16 out
    xn = torch.randn(16384, 8192, device=dev, dtype=torch.float16)
    zn, wn = ri(16384, 8192), torch.ones(8192, device=dev, dtype=torch.float16)
    ms = _time_fn(lambda: ops.qlayer_normgated_fwd(xn, wn, None, 1e-5, q_z=zn, z_scale=0.02, use_float16_output=True, group_size=8192, norm_before_gate=False), steps, warmup)
    nbytes = 16384 * 8192 * (2 + 1 + 2)
    out.append(dict(workload="gated RMS norm, 16384 rows x 8192 (fp16 in, int8 gate, fp16 out)", us=ms * 1e3,
                    tokens_per_s=16384 / ms * 1e3, bound="hbm", achieved_GBs=nbytes / ms / 1e6,
                    frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
    # the same norm in groups of 1024 with the Hadamard transform + quantisation in the same kernel (what the
    # Mamba2-8b mixer runs between the SSD scan and out_proj): fp16 and int8 gate in, int8 out
    ms = _time_fn(lambda: ops.qlayer_normgated_hadamard_quant(xn, wn, 1e-5, 0.2, q_z=zn, z_scale=0.02, group_size=1024,
                                                              norm_before_gate=False), steps, warmup)
    nbytes = 16384 * 8192 * (2 + 1 + 1)
    out.append(dict(workload="gated RMS norm (groups of 1024) + Hadamard + int8 quantisation in one kernel, 16384 rows x 8192",
                    us=ms * 1e3, tokens_per_s=16384 / ms * 1e3, bound="hbm", achieved_GBs=nbytes / ms / 1e6,
                    frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
    del xn, zn, wn
    torch.cuda.empty_cache()
    # the whole Mamba2-8b W4A8 mixer over a prompt (W4A8QMamba2.forward: in_proj, xBC conv, SSD chunk scan, gated
    # norm + Hadamard, out_proj), 16 x 1024 tokens, d_model 4096, 128 heads of 64, d_state 128, 8 groups, chunk 256
    from quamba_amd import W4A8QMamba2
    G = 8
    m2 = W4A8QMamba2(4096, 128, 4, 2, 64, ngroups=G, chunk_size=256, device=dev, state_dtype=torch.float32)
    gen = torch.Generator(device=dev).manual_seed(5)
    for lin, s_ch in ((m2.in_proj, 2e-4), (m2.out_proj, 1e-5)):
        n, k = lin.size_n, lin.size_k
        lin.weight = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=gen)
        lin.s_group = (torch.rand(k // 128, n, device=dev, generator=gen) * 13.8 + 2.0).half()
        lin.s_channel = torch.full((1, n), s_ch, device=dev)
        lin.input_scale = torch.tensor(0.05, device=dev)
    c2 = m2.conv1d
    dim = c2.weight.shape[0]
    c2.weight, c2.bias = ri(dim, 4), ri(dim)
    c2.x_scale = c2.B_scale = c2.C_scale = 0.03
    c2.wx_scale = c2.wB_scale = c2.wC_scale = 0.004
    c2.bx_scale = c2.bB_scale = c2.bC_scale = 0.002
    c2.x_out_scales = torch.full((G, 4, 4), 0.02, device=dev)
    c2.B_out_scales = c2.C_out_scales = torch.full((G,), 0.02, device=dev)
    c2.x_head_group_range = (torch.arange(1, 5, dtype=torch.int32, device=dev) * 4).repeat(G, 1)
    c2.x_dim_group_range = (torch.arange(1, 5, dtype=torch.int32, device=dev) * 16).repeat(G, 4, 1)
    q2 = m2.qchunk_scan
    q2.A_log, q2.D = ri(m2.nheads), ri(m2.nheads)
    q2.dt_bias = torch.full((m2.nheads,), -3.0, dtype=torch.float16, device=dev)
    q2.A_log_scale, q2.D_scale, q2.dt_scale = (torch.tensor(v, device=dev) for v in (0.02, 0.008, 0.02))
    q2.x_scales, q2.B_scale, q2.C_scale = c2.x_out_scales, c2.B_out_scales, c2.C_out_scales
    q2.x_head_group_range, q2.x_dim_group_range = c2.x_head_group_range, c2.x_dim_group_range
    m2.norm.weight = torch.ones(m2.d_ssm, dtype=torch.float16, device=dev)
    m2.norm.z_scale = 0.03
    m2.had.x_H_scale = 0.04
    u2 = ri(16, 1024, 4096)
    ms = _time_fn(lambda: m2.forward(u2), min(steps, 10), 3)
    gemm_ops = 2.0 * 16384 * (4096 * m2.in_proj.size_n + 8192 * 4096)
    out.append(dict(workload="Mamba2-8b W4A8 mixer forward over a prompt (in_proj, conv, SSD scan, norm + Hadamard, out_proj), 16 x 1024 tokens",
                    us=ms * 1e3, tokens_per_s=16384 / ms * 1e3, bound="mfma", achieved_TOPs=gemm_ops / ms / 1e9,
                    frac=gemm_ops / ms / 1e9 / INT8_PEAK_TOPS))
    del u2
    # the same module for one token (W4A8QMamba2.step: in_proj, xBC conv update, state update, norm + Hadamard,
    # out_proj), captured eight times into one HIP graph; bytes = the packed weights + the fp32 state, read and written
    w_bytes = sum(l.weight.numel() + l.s_group.numel() * 2 for l in (m2.in_proj, m2.out_proj))
    for B in (1, 64):
        caches = [m2.allocate_inference_cache(B) for _ in range(8)]
        h1 = ri(B, 1, 4096)

        def token2():
            for cs, ss in caches:
                m2.step(h1, cs, ss)
        for _ in range(3):
            token2()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            token2()
        ms = _time_fn(graph.replay, 64, 4) / len(caches)
        nbytes = w_bytes + B * (2 * m2.nheads * m2.headdim * m2.d_state * 4 + 4096 + 2 * 4096)
        out.append(dict(workload=f"Mamba2-8b W4A8 mixer, one token (five kernels), batch {B}, HIP graph of 8 steps on one layer's weights",
                        us=ms * 1e3, tokens_per_s=B / ms * 1e3, bound="hbm", achieved_GBs=nbytes / ms / 1e6,
                        frac=nbytes / ms / 1e6 / HBM_PEAK_GBS))
        del graph, caches
    return out


def _probes():
    """ctypes handle of the bench-only probe library (bench_probes/libqa_bench_probes.so, built by bench_probes.build)."""
    import ctypes as C
    path = os.path.join(ROOT, "bench_probes", "libqa_bench_probes.so")
    if not os.path.exists(path):
        sys.exit(f"{path} is missing: build it with `python -m bench_probes.build`")
    h = C.CDLL(path)
    vp = C.c_void_p
    for name in ("qa_probe_mfma_i8", "qa_probe_valu"):
        fn = getattr(h, name)
        fn.restype = C.c_int
        fn.argtypes = [vp, C.c_int64, vp, C.c_int, C.c_int, C.c_int, vp]
    return h


def mfma_calibration(dev, kinds=(("constant_operands", 0), ("random_operands", 1)), launches=6):
    """Sustained v_mfma_i32_32x32x32_i8 rate of a register-only loop (two waves per SIMD on every CU) for
    constant and for pseudo-random operand bytes, six launches of about 5 ms each; the last one is reported.
    The clock is the ratio of the shader-clock and 100 MHz counters over the loop."""
    from quamba_amd import _lib
    lib = _probes()
    wgs, iters = 512, 20000
    sink = torch.empty(wgs * 256, dtype=torch.int32, device=dev)
    ticks = torch.zeros(2, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    for name, rnd in kinds:
        for _ in range(launches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.qa_probe_mfma_i8(sink.data_ptr(), sink.numel(), ticks.data_ptr(), wgs, iters, rnd, stream), "diag")
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
        t = ticks.tolist()
        out[name] = {"TOPs": round(8 * 65536.0 * iters * wgs * 4 / ms / 1e9, 1), "ms": round(ms, 3),
                     "clock_MHz": round(100.0 * t[0] / max(t[1], 1), 1)}
    return out


def valu_calibration(dev, ops_list=None, launches=4):
    """Issue time of plain and transcendental vector instructions: eight waves per SIMD on every CU, each lane with
    eight independent chains of one instruction; ns per wave-instruction per SIMD and the clock during the loop."""
    from quamba_amd import _lib
    lib = _probes()
    wgs, iters = 2048, 20000
    sink = torch.empty(wgs * 256, dtype=torch.float32, device=dev)
    ticks = torch.zeros(2, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    simds = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
    out = {}
    all_ops = (("v_mul_f32", 0), ("v_exp_f32", 1), ("v_rcp_f32", 2), ("v_log_f32", 3), ("v_fmac_f32", 4), ("v_mul_f32_dpp", 5))
    for name, op in all_ops:
        if ops_list is not None and name not in ops_list:
            continue
        for _ in range(launches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.qa_probe_valu(sink.data_ptr(), sink.numel(), ticks.data_ptr(), wgs, iters, op, stream), "diag")
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
        t = ticks.tolist()
        per_simd = wgs * 4.0 / simds * iters * 8
        out[name] = {"ns_per_wave_instruction_per_simd": round(ms * 1e6 / per_simd, 3), "ms": round(ms, 3),
                     "clock_MHz": round(100.0 * t[0] / max(t[1], 1), 1)}
    return out


# Vector instructions a wave of the selective scan issues per group of four steps, counted in the compiled kernel
# (time loop + staging of the next tile + output store, divided by the eight groups of a 32-step tile): the kind with
# four lanes per channel and four states per lane, and the short kind with eight lanes per channel and two states.
# The counts belong to one state of the kernel source: `source_sha256` is the hash of quamba_amd/csrc/sscan.hip they
# were counted at; when the file has changed since, the line says so (`stale`) instead of passing them off as current.
SCAN_MIX = {"four_lane": {"plain": 96, "transcendental": 18}, "eight_lane": {"plain": 57, "transcendental": 9}}
SCAN_MIX_SOURCE_SHA256 = "e70cab8ddcf16e14fb332f9d44a854577bfdeee217b5a47359992baa1c18e961"


def scan_mix_is_stale():
    import hashlib
    path = os.path.join(ROOT, "quamba_amd", "csrc", "sscan.hip")
    return hashlib.sha256(open(path, "rb").read()).hexdigest() != SCAN_MIX_SOURCE_SHA256


def peaks_measured(dev):
    """What this GPU sustains right now, beside the published peaks the fractions are quoted against: a plain
    1 GiB device-to-device copy (read + write bytes per second) and the int8 matrix rate of a register-only loop with
    pseudo-random operand bytes (the part lowers its clock under the switching activity of live operands)."""
    src = torch.zeros(1 << 30, dtype=torch.int8, device=dev)
    dst = torch.empty_like(src)
    ms = _time_fn(lambda: dst.copy_(src), 5, 2)
    del src, dst
    torch.cuda.empty_cache()
    m = mfma_calibration(dev, kinds=(("random_operands", 1),), launches=4)["random_operands"]
    return {"copy_GBs": round(2.0 * (1 << 30) / ms / 1e6, 1), "copy_bytes": 1 << 30,
            "int8_mfma_random_operands_TOPs": m["TOPs"], "int8_mfma_clock_MHz": m["clock_MHz"]}


def gemm_phase_clocks(dev, mixer):
    """Where the two projections spend their time and at what clock: the library built with -DQA_GEMM_CLK
    (bench_probes/libquamba_amd_clk.so) has every workgroup record the shader clock and the constant 100 MHz clock at
    the boundaries of its prologue (first operand tiles), main loop and epilogue.  Medians over the workgroups."""
    import ctypes as C
    from quamba_amd import _lib
    path = os.path.join(ROOT, "bench_probes", "libquamba_amd_clk.so")
    if not os.path.exists(path):
        sys.exit(f"{path} is missing: build it with `python -m bench_probes.build`")
    clk = C.CDLL(path)
    clk.qa_gemm_w8a8.restype = C.c_int
    clk.qa_gemm_w8a8.argtypes = [C.POINTER(_lib.QaGemmW8A8Params), C.c_void_p]
    clk.qa_gemm_clk_read.restype = C.c_int
    clk.qa_gemm_clk_read.argtypes = [C.c_void_p, C.c_int64]
    prod = _lib.lib()
    real = prod.qa_gemm_w8a8
    out = {}
    try:
        prod.qa_gemm_w8a8 = clk.qa_gemm_w8a8                       # the modules call through this handle
        for name, fn, m, n, tile in (("in_proj_w8a8_gemm", lambda: mixer.in_proj.to_seqlen_last(mixer.hidden),
                                      2 * mixer.D, mixer.B * mixer.L, (320, 256)),
                                     ("out_proj_w8a8_gemm", lambda: mixer.out_proj(mixer.y_q),
                                      mixer.B * mixer.L, mixer.dm, (256, 320))):
            buf = np.zeros((8192, 8), np.uint64)
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
            clk.qa_gemm_clk_read(buf.ctypes.data_as(C.c_void_p), buf.nbytes)      # clears the table
            ms = _time_fn(fn, 10, 0)
            tiles = -(-m // tile[0]) * -(-n // tile[1])
            if clk.qa_gemm_clk_read(buf.ctypes.data_as(C.c_void_p), buf.nbytes) != 0:
                continue
            b = buf.astype(np.int64)
            b = b[b[:, 0] != 0]                  # one row per workgroup: the last tile it worked on
            wgs = len(b)
            if wgs == 0:
                continue
            dc, dw = np.diff(b[:, 0::2], axis=1), np.diff(b[:, 1::2], axis=1)
            phases = {}
            for i, ph in enumerate(("prologue", "main_loop", "epilogue")):
                phases[ph] = {"us": round(float(np.median(dw[:, i])) / 100.0, 2),
                              "shader_cycles": int(np.median(dc[:, i])),
                              "clock_MHz": round(float(np.median(dc[:, i] / np.maximum(dw[:, i], 1))) * 100.0, 1)}
            out[name] = {"us": round(ms * 1e3, 1), "tiles": tiles, "workgroups": wgs, "tile": list(tile), **phases}
        # the same in_proj launch on operands that switch less: the cycles stay, the clock rises
        zeros = torch.zeros_like(mixer.hidden)
        weight = mixer.in_proj.weight.clone()
        for label, zero_w in (("in_proj_zero_activations", False), ("in_proj_all_operands_zero", True)):
            if zero_w:
                mixer.in_proj.weight.zero_()
            buf = np.zeros((8192, 8), np.uint64)
            for _ in range(10):
                mixer.in_proj.to_seqlen_last(zeros)
            torch.cuda.synchronize()
            clk.qa_gemm_clk_read(buf.ctypes.data_as(C.c_void_p), buf.nbytes)
            ms = _time_fn(lambda: mixer.in_proj.to_seqlen_last(zeros), 10, 0)
            if clk.qa_gemm_clk_read(buf.ctypes.data_as(C.c_void_p), buf.nbytes) == 0:
                b = buf.astype(np.int64)
                b = b[b[:, 0] != 0]
                dc, dw = np.diff(b[:, 0::2], axis=1), np.diff(b[:, 1::2], axis=1)
                out[label] = {"us": round(ms * 1e3, 1),
                              "main_loop": {"us": round(float(np.median(dw[:, 1])) / 100.0, 2), "shader_cycles": int(np.median(dc[:, 1])),
                                            "clock_MHz": round(float(np.median(dc[:, 1] / np.maximum(dw[:, 1], 1))) * 100.0, 1)}}
        mixer.in_proj.weight.copy_(weight)
    finally:
        prod.qa_gemm_w8a8 = real
    return out


def scan_mix_rates(dev, waves_per_simd=8):
    """Issue time of the scan's own instruction mix on live values (probe ops 6 and 7: the recurrence on registers,
    four plain instructions and one exp2 per chain step, and the same with four more plain instructions): ns per
    plain and per transcendental wave-instruction per SIMD, and the clock the part settles at under that activity,
    with `waves_per_simd` resident waves on every SIMD (eight: what the vector ALUs sustain; fewer: what that many
    waves can draw from them).  Constant operands (valu_calibration) leave the part at its highest clock and give
    lower figures."""
    from quamba_amd import _lib
    lib = _probes()
    simds = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
    wgs, iters = waves_per_simd * simds // 4, 10000
    sink = torch.empty(wgs * 256, dtype=torch.float32, device=dev)
    ticks = torch.zeros(2, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    ns, clock = {}, {}
    for op in (6, 7):
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.qa_probe_valu(sink.data_ptr(), sink.numel(), ticks.data_ptr(), wgs, iters, op, stream), "diag")
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
        t = ticks.tolist()
        ns[op] = ms * 1e6 / (wgs * 4.0 / simds * iters * 8)       # per chain step per SIMD
        clock[op] = 100.0 * t[0] / max(t[1], 1)
    t_plain = (ns[7] - ns[6]) / 4.0
    return dict(ns_plain=t_plain, ns_transcendental=ns[6] - 4.0 * t_plain, clock_MHz=clock[6])


def scan_issue_bound(dev, B, D, L):
    """Lower bound of the scan launch from vector-ALU issue alone: every wave's instruction mix priced at the rates
    the same mix reaches in a register-only loop on live values on this GPU now (scan_mix_rates), the waves spread
    evenly over the SIMDs.  The split into the two kinds of workgroup is the library's own (qa_sscan_chosen_mapping).
    `issue_bound_us` uses the rates of eight resident waves per SIMD (what the vector ALUs sustain);
    `issue_bound_at_launch_occupancy_us` uses the rates the probe reaches with as many waves per SIMD as this launch
    has - a single wave cannot issue back to back, so few waves draw less from the same ALUs."""
    simds = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
    lanes, arg = ops.sscan_chosen_mapping(B, D, CFG["d_state"])
    short = D if lanes == 8 else (D - 64 * arg if lanes == 0 else 0)
    waves = {"four_lane": B * (D - short) // 16, "eight_lane": B * short // 8}
    groups = (L + 31) // 32 * 8
    wps = -(-(waves["four_lane"] + waves["eight_lane"]) // simds)
    out = dict(waves=waves, waves_per_simd=wps, instructions_per_four_steps=SCAN_MIX, stale=scan_mix_is_stale())
    for key, n in (("issue_bound_us", 8), ("issue_bound_at_launch_occupancy_us", wps)):
        rates = scan_mix_rates(dev, n)
        t_plain, t_trans = rates["ns_plain"], rates["ns_transcendental"]
        ns = sum(waves[k] * groups * (SCAN_MIX[k]["plain"] * t_plain + SCAN_MIX[k]["transcendental"] * t_trans) for k in waves)
        out[key] = ns / simds / 1e3
        out[key.replace("_us", "_rates")] = dict(ns_plain=round(t_plain, 3), ns_transcendental=round(t_trans, 3),
                                                 clock_MHz=round(rates["clock_MHz"], 1), waves_per_simd=n)
    return out


def load_traffic(path):
    """HBM bytes per launch from the rocprofv3 counter runs summarised in profiles/hbm_traffic_counters.md: the file
    names the git head it was measured at and, per entry, the kernels it sums.  An entry whose kernels no longer exist
    in the library under those names is dropped (its figure would belong to other code)."""
    if not os.path.exists(path):
        return {}, None
    from quamba_amd import _lib
    doc = json.load(open(path))
    image = open(_lib.LIB_PATH, "rb").read()
    out = {}
    for name, entry in doc.get("entries", {}).items():
        if all(sym.encode() in image for sym in entry["kernel_symbols"]):
            out[name] = entry["bytes"]
    return out, doc.get("head")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=CFG["batch"])
    ap.add_argument("--seqlen", type=int, default=CFG["seqlen"])
    ap.add_argument("--input-sets", type=int, default=3,
                    help="step i reads input set i %% N (hidden states, dt, B, C, out_proj input at other addresses)")
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="untimed repetitions of the step before the warm-up steps, for this long, so that the part's "
                         "clocks have settled on the workload (0: none)")
    ap.add_argument("--runs", type=int, default=5,
                    help="timed runs of --steps steps each; the line's value is the first, the others give the median and spread")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="leave out the short list of the other benchmark configurations (decode step, Mamba2-2.7b SSD "
                         "scan, Mamba2-8b in_proj / SSD scan / out_proj)")
    ap.add_argument("--other-workloads", action="store_true",
                    help="also time the long list: whole mixers, Mamba2 conv, Hadamard, norms, single-token W4A8 "
                         "(key other_workloads_long in the JSON line)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies (reference points for hardware-counter runs)")
    ap.add_argument("--mfma-calibration", action="store_true",
                    help="also measure the int8 matrix rate the part sustains in a register-only loop, with constant and "
                         "with random operand bytes (extra key in the JSON line)")
    ap.add_argument("--valu-calibration", action="store_true",
                    help="also measure the issue time of plain and transcendental vector instructions (extra key in the JSON line)")
    ap.add_argument("--gemm-phase-clocks", action="store_true",
                    help="also report, for both projections, the time and the clock of a workgroup's prologue, main loop "
                         "and epilogue (needs bench_probes/libquamba_amd_clk.so)")
    ap.add_argument("--traffic-json", default=os.path.join(ROOT, "profiles", "traffic.json"),
                    help="HBM bytes per launch measured with rocprofv3 --pmc, with the git head and the kernel names they "
                         "were measured at")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU only: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    global SETTLE_MS
    SETTLE_MS = min(SETTLE_MS, max(0.0, args.settle_ms))
    mixer = Mixer(dev, args.batch, args.seqlen, input_sets=max(1, args.input_sets))
    B, L = args.batch, args.seqlen

    # Settling: the part's power management needs about 30 ms of a new workload to converge (a cold start runs its
    # first steps fast, is throttled below its steady clock for the next ten, and climbs back over twenty more: the scan
    # goes 462, 519, 545, 545, 512, 476 ... 430 (step 14) ... 410 us (step 28)).  The mixer step is therefore repeated,
    # untimed, for --settle-ms before the W warm-up steps; `settle_steps` in the line says how often.
    DOM = 2
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]     # before any GPU work:
    settle_steps = 0                                                 # creating them later would leave the GPU idle
    if args.settle_ms > 0:
        torch.cuda.synchronize()
        t_settle = time.perf_counter()
        mixer.step()
        torch.cuda.synchronize()
        est_ms = max((time.perf_counter() - t_settle) * 1e3, 0.05)
        t_settle = time.perf_counter()
        mixer.step()
        torch.cuda.synchronize()
        est_ms = min(est_ms, max((time.perf_counter() - t_settle) * 1e3, 0.05))
        settle_steps = 2 + int(min(2000, max(0.0, args.settle_ms / est_ms)))
        for _ in range(settle_steps - 2):            # queued back to back, no host synchronisation in between
            mixer.step()
    for _ in range(args.warmup):
        mixer.step()
    torch.cuda.synchronize()
    # The timed region: K steps, with HIP events around the dominant kernel only (the selective scan, position 2..3).
    # An event between two kernels is a marker that waits for the kernel before it, so the events around the other three
    # kernels are left to a pass of their own after the timed runs.
    t0 = time.perf_counter()
    for i in range(args.steps):
        mixer.step(ev[i], only=(DOM, DOM + 1))
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    dom_us_timed = float(np.mean([ev[i][DOM].elapsed_time(ev[i][DOM + 1]) for i in range(args.steps)])) * 1e3
    # the same K steps again, runs - 1 times, without events: median and spread of the per-step time (the line's value
    # stays the first run)
    run_ms = [ms_per_step]
    for _ in range(max(0, args.runs - 1)):
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(args.steps):
            mixer.step()
        torch.cuda.synchronize()
        run_ms.append((time.perf_counter() - t1) * 1e3 / args.steps)
    # per-kernel pass: K more steps with events between all kernels (its own per-step time is reported beside the table)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for i in range(args.steps):
        mixer.step(ev[i])
    torch.cuda.synchronize()
    kernels_pass_ms = (time.perf_counter() - t2) * 1e3 / args.steps

    kernels = kernel_table(B, L)
    for j, kinfo in enumerate(kernels):
        dur_ms = float(np.mean([ev[i][j].elapsed_time(ev[i][j + 1]) for i in range(args.steps)]))
        if j == DOM:
            kinfo["avg_us_kernels_pass"] = dur_ms * 1e3
            dur_ms = dom_us_timed / 1e3                 # the dominant kernel's figure is the timed region's
        kinfo["avg_us"] = dur_ms * 1e3
        if kinfo["bound"] == "hbm":
            kinfo.update(achieved=kinfo["bytes"] / dur_ms / 1e6, peak=HBM_PEAK_GBS, unit="GB/s")
        else:
            kinfo.update(achieved=kinfo["ops"] / dur_ms / 1e9, peak=INT8_PEAK_TOPS, unit="TOP/s")
        kinfo["frac"] = kinfo["achieved"] / kinfo["peak"]
    traffic, traffic_head = load_traffic(args.traffic_json)
    dom = kernels[DOM] if kernels[DOM]["avg_us"] >= 0.9 * max(k["avg_us"] for k in kernels) else max(kernels, key=lambda k: k["avg_us"])
    roofline = dict(kernel=dom["name"], bound=dom["bound"], achieved=round(dom["achieved"], 2), peak=dom["peak"],
                    unit=dom["unit"], frac=round(dom["frac"], 4), traffic=traffic.get(dom["name"]),
                    traffic_head=traffic_head, avg_us=round(dom["avg_us"], 2))
    if dom["name"] == "sscan_fwd":
        # the bound that binds this kernel is vector-ALU issue, not HBM: how far the launch is from it
        ib = scan_issue_bound(dev, B, CFG["d_inner"], L)
        if ib["stale"]:
            roofline["issue_bound_stale"] = "quamba_amd/csrc/sscan.hip has changed since the instruction mix was counted"
        else:
            roofline["issue_bound_us"] = round(ib["issue_bound_us"], 2)
            roofline["frac_of_issue_bound"] = round(ib["issue_bound_us"] / dom["avg_us"], 4)
            roofline["issue_bound_at_launch_occupancy_us"] = round(ib["issue_bound_at_launch_occupancy_us"], 2)
            roofline["frac_of_issue_bound_at_launch_occupancy"] = round(ib["issue_bound_at_launch_occupancy_us"] / dom["avg_us"], 4)
        roofline["issue_bound_inputs"] = {k: ib[k] for k in ("issue_bound_rates", "issue_bound_at_launch_occupancy_rates",
                                                             "waves", "waves_per_simd", "instructions_per_four_steps")}
    per_kernel = [dict(kernel=k["name"], bound=k["bound"], avg_us=round(k["avg_us"], 2), achieved=round(k["achieved"], 2),
                       unit=k["unit"], peak=k["peak"], frac=round(k["frac"], 4), traffic=traffic.get(k["name"]),
                       measured_in="timed region" if "avg_us_kernels_pass" in k else "kernels pass",
                       **({"avg_us_kernels_pass": round(k["avg_us_kernels_pass"], 2)} if "avg_us_kernels_pass" in k else {}))
                  for k in kernels]

    line = {
        "metric": "quantized mixer prefill tokens/s on 1 MI355X; % HBM peak (scan) / % int8 MFMA (GEMM)",
        "value": round(B * L / (ms_per_step / 1e3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_runs": [round(v, 4) for v in run_ms],
        "ms_per_step_median": round(float(np.median(run_ms)), 4),
        "input_sets": len(mixer.sets),
        "settle_steps": settle_steps,
        "kernels_pass_ms_per_step": round(kernels_pass_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "Mamba1-2.8b quantized prefill mixer: in_proj W8A8 -> conv1d int8 -> selective scan int8 "
                               "(z gate, fp16 out, fp32 state) -> out_proj W8A8",
                   "batch": B, "seq_len": L, "d_model": CFG["d_model"], "d_inner": CFG["d_inner"],
                   "d_state": CFG["d_state"], "d_conv": CFG["d_conv"], "tokens_per_step": B * L},
        "roofline": roofline,
        "kernels": per_kernel,
    }
    # after the timed runs: a burst of matrix instructions at the power limit right before them depresses the clock of
    # the steps that follow for longer than the settling phase lasts
    line["peaks_measured"] = peaks_measured(dev)
    if args.gemm_phase_clocks:
        line["gemm_phase_clocks"] = gemm_phase_clocks(dev, mixer)
    if args.copy_calibration:
        src = torch.zeros(1 << 30, dtype=torch.int8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.mfma_calibration:
        line["mfma_calibration"] = mfma_calibration(dev)
    if args.valu_calibration:
        line["valu_calibration"] = valu_calibration(dev)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(mixer)
    del mixer
    torch.cuda.empty_cache()
    rounded = lambda ws: [{k: (round(v, 4) if isinstance(v, float) else v) for k, v in w.items()} for w in ws]
    if not args.no_other_workloads:
        ws = secondary_workloads(dev, min(args.steps, 20), args.warmup)
        for w in ws:
            w["traffic"] = traffic.get(w["name"])
        line["other_workloads"] = rounded(ws)
    if args.other_workloads:
        line["other_workloads_long"] = rounded(other_workloads(dev, min(args.steps, 20), args.warmup))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
