#!/usr/bin/env python3
"""Benchmark of the FractalTensor hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload b2b|config1|attention|stacked_lstm|dilated_lstm|...]
                    [--no-extras] [--all] [--no-cpu] [--no-baselines]

Prints ONE JSON line.  The headline workload is BASELINE.json configs[1], the
fused back-to-back fp16 GEMM (32 problems of [4096,128]x[128,128]x[128,128]);
the other configurations (the single-layer scan with the host's eager operator
program beside it, flash attention, stacked LSTM, dilated LSTM) are measured
the same way and reported under "other_workloads" unless --no-extras is given,
and summarised in "configs", the last key of the line.  --all adds the
workloads either side of the path.  A step is one pass of the kernel over one batch of
synthetic input that is already resident in HBM.  For the B2B GEMM the timed
steps walk a ring of input sets larger than the 256 MB memory-side cache, so
the figure is an HBM figure; the same-buffers figure is reported next to it.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# BASELINE.json configs[i] -> key of the compact per-configuration summary
CONFIG_OF = {'config1': 'configs[0]', 'b2b': 'configs[1]', 'attention': 'configs[2]', 'stacked_lstm': 'configs[3]', 'dilated_lstm': 'configs[4]'}

# MI355X published peaks (dense)
PEAK_HBM_GBS = 8000.0
PEAK_F16_TFLOPS = 2500.0
PEAK_F32_MATRIX_TFLOPS = 157.3

# HBM traffic per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (profiles/*_pmc.txt name the commands); None = not measured for that kernel.
MEASURED_TRAFFIC_BYTES = {}
try:
    with open(os.path.join(ROOT, 'profiles', 'traffic.json')) as _f:
        MEASURED_TRAFFIC_BYTES = json.load(_f)
except Exception:
    pass


def _events_ms(torch, fn, steps, warmup):
    """Average duration of fn over `steps` launches, HIP events on the launch stream.  After the warm-up and the
    synchronisation a spin kernel of about 0.1 ms runs ahead of the start event, so that the timed launches are
    queued behind it by the time the device reaches the event: what is timed is the device working through `steps`
    launches back to back, not the idle-to-busy latency of the first launch after a synchronisation (about 10 us,
    which is 3 % of a region of twenty 17 us launches)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    torch.cuda._sleep(200000)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(end) / steps, wall


def _host_threads():
    """Threads for the host legs: the physical cores, capped at the 16 a one-GPU box gives a job."""
    try:
        import psutil
        n = psutil.cpu_count(logical=False) or os.cpu_count() or 1
    except Exception:
        n = os.cpu_count() or 1
    return max(1, min(16, n))


def _host_timed(torch, fn, warm, runs):
    """(last result, median seconds, min seconds, threads) of fn on torch CPU with torch.set_num_threads(physical
    cores, at most 16): the way every torch-CPU baseline of this file is timed."""
    threads = _host_threads()
    before = torch.get_num_threads()
    torch.set_num_threads(threads)
    try:
        for _ in range(warm):
            out = fn()
        t = []
        for _ in range(runs):
            t0 = time.perf_counter()
            out = fn()
            t.append(time.perf_counter() - t0)
    finally:
        torch.set_num_threads(before)
    return out, sorted(t)[len(t) // 2], min(t), threads


def _lstm_torch_cpu(torch, xs, WU, dil=None):
    """The batched LSTM loop on torch CPU: per layer and step one [B, 2H] @ [2H, 4H] product and the gate arithmetic
    as torch operators (the batched form of examples/stacked_rnn/stacked_rnn.py:23-65 and of
    benchmarks/rnn/baselines/stacked_lstm/pt_model/rnn.py:94-108).  Returns every layer's h, a list of [T, B, H]."""
    L = WU.shape[0]
    T, B, H = xs.shape
    inp = xs
    layers = []
    for l in range(L):
        d = 1 if dil is None else dil[l]
        hs, cs = [], []
        zero = torch.zeros((B, H))
        for t in range(T):
            h, c = (hs[t - d], cs[t - d]) if t >= d else (zero, zero)
            g = torch.cat([inp[t], h], dim=1) @ WU[l]
            i, f, o, cand = g.chunk(4, 1)
            c = torch.sigmoid(f) * c + torch.sigmoid(i) * torch.tanh(cand)
            h = torch.sigmoid(o) * torch.tanh(c)
            hs.append(h)
            cs.append(c)
        inp = torch.stack(hs)
        layers.append(inp)
    return layers


def bench_b2b(torch, core, steps, warmup, cpu):
    G, M, N, K, P = 32, 4096, 128, 128, 128
    flop = 2.0 * G * M * N * (K + P)
    nbytes = 2.0 * G * (M * K + N * K + P * N + M * P)
    gen = torch.Generator(device='cpu').manual_seed(1234)
    ring = 8   # 8 x 69 MB of operands and results: larger than the 256 MB memory-side cache
    sets = []
    for _ in range(ring):
        A = (torch.randn((G, M, K), generator=gen) / K ** 0.5).half().cuda()
        Bn = (torch.randn((G, N, K), generator=gen) / K ** 0.5).half().cuda()
        Cp = (torch.randn((G, P, N), generator=gen) / N ** 0.5).half().cuda()
        D = torch.empty((G, M, P), dtype=torch.float16, device='cuda')
        sets.append((A, Bn, Cp, D))
    state = {'i': 0}

    def step_ring():
        A, Bn, Cp, D = sets[state['i'] % ring]
        state['i'] += 1
        core.b2b_gemm(A, Bn, Cp, out=D)

    def step_same():
        A, Bn, Cp, D = sets[0]
        core.b2b_gemm(A, Bn, Cp, out=D)

    ms, wall = _events_ms(torch, step_ring, steps, warmup)
    ms_same, _ = _events_ms(torch, step_same, steps, warmup)
    res = {
        'metric': 'TFLOP/s + % MFMA peak (B2B GEMM)',
        'value': flop / ms / 1e9, 'unit': 'TFLOP/s', 'ms_per_step': ms, 'dtype': 'f16',
        'config': {'workload': 'fused back-to-back GEMM D=(A@B)@C, BASELINE.json configs[1]',
                   'problems': G, 'M': M, 'N': N, 'K': K, 'P': P, 'accumulate': 'f32',
                   'inputs': 'ring of 8 operand sets (553 MB) so steps read HBM, not the memory-side cache'},
        'pct_f16_mfma_peak': 100.0 * flop / ms / 1e9 / PEAK_F16_TFLOPS,
        'same_buffers': {'ms_per_step': ms_same, 'tflops': flop / ms_same / 1e9, 'gbs': nbytes / ms_same / 1e6},
        'host_wall_ms_per_step': wall,
        'roofline': {'bound': 'hbm', 'achieved': nbytes / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                     'frac': nbytes / ms / 1e6 / PEAK_HBM_GBS,
                     'traffic': MEASURED_TRAFFIC_BYTES.get('b2b_gemm8_kernel'),
                     'kernel': 'b2b_gemm8_kernel<8,4,4>', 'algorithmic_bytes_per_launch': nbytes},
    }
    if cpu:
        # the frontend's own eager expression, (a @ b) @ c per problem, on torch CPU.  fp32 operands (the fp16 values,
        # widened beforehand): torch's host GEMM is built for fp32, so this is the host at its best, not at its worst
        from fractaltensor_amd.kaleido import Tensor
        A, Bn, Cp, _ = sets[0]
        a32, b32, c32 = A.float().cpu(), Bn.transpose(1, 2).float().cpu().contiguous(), Cp.transpose(1, 2).float().cpu().contiguous()
        ta, tb, tc = ([Tensor.from_tensor(x[g]) for g in range(G)] for x in (a32, b32, c32))
        eager = lambda: [(ta[g] @ tb[g]) @ tc[g] for g in range(G)]
        out, med, best, threads = _host_timed(torch, eager, 2, 10)
        core.b2b_gemm(A, Bn, Cp, out=sets[0][3])
        diff = float((out[G - 1].data - sets[0][3][G - 1].float().cpu()).abs().max() / out[G - 1].data.abs().max())
        assert diff <= 1e-2, diff
        res['cpu_baseline'] = {'value': flop / med / 1e12, 'unit': 'TFLOP/s', 'cores': threads, 'kind': 'torch_cpu_eager',
                               'sample': f'the whole configuration: the operator expression (a @ b) @ c of the frontend on the {G} '
                                         f'problems in turn, fp32 torch CPU tensors, torch.set_num_threads({threads}) of '
                                         f'{os.cpu_count()} host CPUs, 2 warm-up + 10 timed runs, median {med * 1e3:.1f} ms '
                                         f'(min {best * 1e3:.1f} ms)',
                               'ms_per_step': med * 1e3, 'max_rel_diff_vs_gpu': diff}
        from oracle import c_oracle
        sample = 8    # a quarter of the problems: a few seconds of scalar C
        a, b, c = (x[:sample].cpu().numpy() for x in (A, Bn, Cp))
        t0 = time.perf_counter()
        c_oracle.b2b_gemm(a, b, c, round_intermediate=True)
        dt = time.perf_counter() - t0
        res['cpu_baseline']['scalar_c_port'] = {'value': flop * sample / G / dt / 1e12, 'unit': 'TFLOP/s', 'cores': 1,
                                                'sample': f'{sample} of the {G} problems through oracle/oracle.c (scalar C, one '
                                                          f'thread), {dt:.1f} s'}
    return res


def _graph_us(torch, fn, calls=20, replays=10):
    """Microseconds per call of fn with the calls replayed from a HIP graph: what is left is the device's own
    kernel-to-kernel cost, not the host's launch path (these kernels are shorter than a ctypes call)."""
    fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(replays):
        graph.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / (calls * replays) * 1e3


def bench_b2b_reference_shapes(torch, core, steps, warmup, cpu):
    """The four shapes of the reference's own B2B benchmark, [8192 | 16384, 64] x [64, 256 | 512] x [., 64]
    (benchmarks/fused_two_hgemms/fractaltensor/fused_two_hgemms.cu:152-175), timed as it times them: the same
    operands again and again (2 to 4.5 MB, so they stay in the caches), here replayed from a HIP graph."""
    gen = torch.Generator(device='cpu').manual_seed(1234)
    shapes = {}
    for M in (8192, 16384):
        for N in (256, 512):
            K = P = 64
            A = (torch.randn((1, M, K), generator=gen) / K ** 0.5).half().cuda()
            Bn = (torch.randn((1, N, K), generator=gen) / K ** 0.5).half().cuda()
            Cp = (torch.randn((1, P, N), generator=gen) / N ** 0.5).half().cuda()
            D = torch.empty((1, M, P), dtype=torch.float16, device='cuda')
            us = _graph_us(torch, lambda: core.b2b_gemm(A, Bn, Cp, out=D))
            Bt, Ct = Bn[0].t().contiguous(), Cp[0].t().contiguous()
            Pm = torch.empty((M, N), dtype=torch.float16, device='cuda')
            D2 = torch.empty((M, P), dtype=torch.float16, device='cuda')
            us_t = _graph_us(torch, lambda: (torch.mm(A[0], Bt, out=Pm), torch.mm(Pm, Ct, out=D2)))
            flop = 2.0 * M * N * (K + P)
            diff = float((D[0].float() - D2.float()).abs().max() / D2.float().abs().max())
            assert diff <= 1e-2, diff
            shapes[f'M{M}_N{N}'] = {'us_per_call': us, 'tflops': flop / us / 1e6, 'two_torch_gemms_us': us_t,
                                    'speedup': us_t / us, 'max_rel_diff_vs_two_gemms': diff,
                                    'bytes': 2.0 * (M * K + N * K + P * N + M * P)}
    top = shapes['M16384_N512']
    flop = 2.0 * 16384 * 512 * 128
    return {'metric': 'TFLOP/s (B2B GEMM, reference benchmark shapes)', 'value': top['tflops'], 'unit': 'TFLOP/s',
            'ms_per_step': top['us_per_call'] / 1e3, 'dtype': 'f16',
            'config': {'workload': 'fused back-to-back GEMM on the reference benchmark shapes, operands resident in the caches, '
                                   'launches replayed from a HIP graph; headline figures are the largest shape (M 16384, N 512)',
                       'K': 64, 'P': 64, 'accumulate': 'f32'},
            'roofline': {'bound': 'mfma', 'achieved': top['tflops'], 'peak': PEAK_F16_TFLOPS, 'unit': 'TFLOP/s',
                         'frac': top['tflops'] / PEAK_F16_TFLOPS, 'traffic': None, 'kernel': 'b2b_wide_kernel<4, 2, 2, 8>',
                         'note': '2.1 GFLOP and 4.5 MB per launch: a launch of a few microseconds, bounded by the kernel-to-kernel '
                                 'cost of the device and the read of B and C by every workgroup, not by the matrix rate'},
            'shapes': shapes}


def bench_copy(torch, core, steps, warmup, cpu):
    """Plain device copy of a known size: the calibration kernel for the FETCH_SIZE / WRITE_SIZE counters."""
    n = 64 << 20   # 64 MiB read + 64 MiB written per launch
    src = torch.empty(n, dtype=torch.uint8, device='cuda').random_()
    dst = torch.empty_like(src)
    ms, _ = _events_ms(torch, lambda: dst.copy_(src), steps, warmup)
    return {'metric': 'copy GB/s (counter calibration)', 'value': 2.0 * n / ms / 1e6, 'unit': 'GB/s', 'ms_per_step': ms,
            'dtype': 'u8', 'config': {'workload': 'torch copy_ of 64 MiB (reads 64 MiB, writes 64 MiB per launch)'},
            'roofline': {'bound': 'hbm', 'achieved': 2.0 * n / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                         'frac': 2.0 * n / ms / 1e6 / PEAK_HBM_GBS, 'traffic': None}}


def bench_attention(torch, core, steps, warmup, cpu):
    B, Hd, S, D = 8, 16, 2048, 128
    flop = 4.0 * B * Hd * S * S * D
    gen = torch.Generator(device='cpu').manual_seed(1234)
    Q, K, V = (torch.randn((B, Hd, S, D), generator=gen).half().cuda() for _ in range(3))
    O = torch.empty_like(Q)
    scale = D ** -0.5
    ms, wall = _events_ms(torch, lambda: core.flash_attention(Q, K, V, scale, out=O), steps, warmup)
    res = {
        'metric': 'TFLOP/s + % MFMA peak (attention)', 'value': flop / ms / 1e9, 'unit': 'TFLOP/s',
        'ms_per_step': ms, 'dtype': 'f16',
        'config': {'workload': 'flash attention, non-causal, BASELINE.json configs[2]', 'batch': B, 'heads': Hd,
                   'seq': S, 'head_dim': D, 'accumulate': 'f32'},
        'pct_f16_mfma_peak': 100.0 * flop / ms / 1e9 / PEAK_F16_TFLOPS,
        'roofline': {'bound': 'mfma', 'achieved': flop / ms / 1e9, 'peak': PEAK_F16_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': flop / ms / 1e9 / PEAK_F16_TFLOPS,
                     'traffic': MEASURED_TRAFFIC_BYTES.get('flash_attn_pp_kernel'), 'kernel': 'flash_attn_pp_kernel'},
    }
    if cpu:
        # the blockwise program of examples/flash_attention/flash_attention.py:14-91 as this package states it
        # (programs.flash_attention: map over samples and heads, map over query blocks, reduce over key blocks of 64
        # rows), eager on torch CPU in fp32 (the example's own element type), on a bounded sample of heads
        from fractaltensor_amd import programs
        from fractaltensor_amd.kaleido import FractalTensor
        heads, blk = 4, 64
        mk = lambda t: FractalTensor.from_dense(t[0:1, :heads].float().cpu().reshape(1, heads, S // blk, blk, D).contiguous(), 3)
        q, k, v = mk(Q), mk(K), mk(V)
        out, med, best, threads = _host_timed(torch, lambda: programs.flash_attention(q, k, v, scale), 0, 2)
        core.flash_attention(Q, K, V, scale, out=O)
        ref = O[0, :heads].float().cpu()
        diff = float((out.as_dense().reshape(heads, S, D) - ref).abs().max() / ref.abs().max())
        assert diff <= 1e-2, diff
        res['cpu_baseline'] = {'value': flop * heads / (B * Hd) / med / 1e12, 'unit': 'TFLOP/s', 'cores': threads,
                               'kind': 'torch_cpu_eager',
                               'sample': f'{heads} of {B * Hd} (batch, head) pairs: the eager operator program '
                                         f'(programs.flash_attention, {S // blk} x {S // blk} blocks of {blk} rows per head) on '
                                         f'fp32 torch CPU tensors, torch.set_num_threads({threads}) of {os.cpu_count()} host CPUs, '
                                         f'2 timed runs, median {med:.2f} s',
                               'max_rel_diff_vs_gpu': diff}
        # the same attention as one torch call per head on the host, to separate operator dispatch from host arithmetic
        qh, kh, vh = (x[0].float().cpu() for x in (Q, K, V))
        sdpa = lambda: torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, scale=scale)
        _, med_s, _, _ = _host_timed(torch, sdpa, 1, 3)
        res['cpu_baseline']['batched'] = {'value': flop / B / med_s / 1e12, 'unit': 'TFLOP/s', 'ms_per_step': med_s * 1e3,
                                          'what': f'torch scaled_dot_product_attention on the {Hd} heads of one sample, fp32, {threads} threads'}
        from oracle import c_oracle
        hs = 4
        q, k, v = (x[0, :hs].cpu().numpy() for x in (Q, K, V))
        t0 = time.perf_counter()
        c_oracle.flash_attention(q, k, v, scale, block_kv=64)
        dt = time.perf_counter() - t0
        res['cpu_baseline']['scalar_c_port'] = {'value': flop * hs / (B * Hd) / dt / 1e12, 'unit': 'TFLOP/s', 'cores': 1,
                                                'sample': f'{hs} of {B * Hd} (batch, head) pairs through oracle/oracle.c, {dt:.1f} s'}
    return res


def bench_attention_few_queries(torch, core, steps, warmup, cpu):
    """Few queries against many keys (a step of decoding with a block of 128 queries): 8 heads x 128 queries x 32768
    keys, D 128, fp16.  Eight workgroups without a split over the keys; with it the grid fills the chip."""
    B, Hd, Sq, Skv, D = 1, 8, 128, 32768, 128
    flop = 4.0 * B * Hd * Sq * Skv * D
    gen = torch.Generator(device='cpu').manual_seed(1234)
    Q = torch.randn((B, Hd, Sq, D), generator=gen).half().cuda()
    K, V = (torch.randn((B, Hd, Skv, D), generator=gen).half().cuda() for _ in range(2))
    O = torch.empty_like(Q)
    scale = D ** -0.5
    ws = torch.empty(int(core.lib.ftk_flash_attn_f16_workspace_bytes(B, Hd, Sq, Skv, D)), dtype=torch.uint8, device='cuda')
    ms, _ = _events_ms(torch, lambda: core.flash_attention(Q, K, V, scale, out=O, workspace=ws), steps, warmup)
    ref = O.clone()
    ms_one, _ = _events_ms(torch, lambda: core.flash_attention(Q, K, V, scale, out=O, split_keys=False), max(3, steps // 4), 1)
    diff = float((O.float() - ref.float()).abs().max() / ref.float().abs().max())
    ms_t, _ = _events_ms(torch, lambda: torch.nn.functional.scaled_dot_product_attention(Q, K, V, scale=scale), max(3, steps // 4), 1)
    nbytes = 2.0 * (2 * B * Hd * Skv * D + 2 * B * Hd * Sq * D)
    return {'metric': 'TFLOP/s (attention, few queries)', 'value': flop / ms / 1e9, 'unit': 'TFLOP/s', 'ms_per_step': ms, 'dtype': 'f16',
            'config': {'workload': 'flash attention split over the keys', 'batch': B, 'heads': Hd, 'queries': Sq, 'keys': Skv, 'head_dim': D},
            'roofline': {'bound': 'hbm', 'achieved': nbytes / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s', 'frac': nbytes / ms / 1e6 / PEAK_HBM_GBS,
                         'traffic': None, 'kernel': 'flash_attn_kernel<128,1,4,1,false,true,true> + attn_merge_kernel<128>',
                         'algorithmic_bytes_per_launch': nbytes, 'note': '128 MB of K and V read once for 137 GFLOP: AI 1024 FLOP/B, but a launch of '
                         'tens of microseconds; K and V of this size stay in the 256 MB memory-side cache between steps'},
            'single_launch': {'ms_per_step': ms_one, 'speedup_of_split': ms_one / ms, 'max_rel_diff': diff},
            'torch_sdpa': {'ms_per_step': ms_t, 'speedup': ms_t / ms}}


def bench_attention_f32(torch, core, steps, warmup, cpu):
    """BASELINE configs[2]'s shape with fp32 Q, K, V, O (the element type of the reference's own attention program):
    every product as three fp16 MFMAs of split operands.  The timed step is the whole entry point: the largest
    |K|, |V| per head, the split of Q, K and V into planes, the attention kernel."""
    B, Hd, S, D = 8, 16, 2048, 128
    flop = 4.0 * B * Hd * S * S * D
    gen = torch.Generator(device='cpu').manual_seed(1234)
    Q, K, V = (torch.randn((B, Hd, S, D), generator=gen).cuda() for _ in range(3))
    O = torch.empty_like(Q)
    ws = torch.empty(int(core.lib.ftk_flash_attn_f32_workspace_bytes(B, Hd, S, S, D)), dtype=torch.uint8, device='cuda')
    scale = D ** -0.5
    ms, _ = _events_ms(torch, lambda: core.flash_attention_f32(Q, K, V, scale, out=O, workspace=ws), steps, warmup)
    ms_t, _ = _events_ms(torch, lambda: torch.nn.functional.scaled_dot_product_attention(Q, K, V, scale=scale), max(2, steps // 4), 1)
    ref = torch.nn.functional.scaled_dot_product_attention(Q[:1].double(), K[:1].double(), V[:1].double(), scale=scale)
    res = {
        'metric': 'TFLOP/s (attention, fp32 data)', 'value': flop / ms / 1e9, 'unit': 'TFLOP/s', 'ms_per_step': ms,
        'dtype': 'f32 (products as three f16 MFMAs of split operands, f32 accumulate)',
        'config': {'workload': 'flash attention, non-causal, fp32 Q/K/V/O at the shape of BASELINE.json configs[2]', 'batch': B,
                   'heads': Hd, 'seq': S, 'head_dim': D},
        'roofline': {'bound': 'mfma', 'achieved': 3 * flop / ms / 1e9, 'peak': PEAK_F16_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': 3 * flop / ms / 1e9 / PEAK_F16_TFLOPS, 'traffic': None, 'kernel': 'flash_attn_f32_kernel<128>',
                     'what': 'MFMA flops issued (three f16 products per fp32 product) against the f16 MFMA peak; the step also '
                             'holds the three launches that split the operands',
                     'algorithmic': {'tflops': flop / ms / 1e9, 'ratio_to_f32_matrix_peak': flop / ms / 1e9 / PEAK_F32_MATRIX_TFLOPS}},
        'torch_sdpa_f32': {'ms_per_step': ms_t, 'speedup': ms_t / ms},
        'max_rel_diff_vs_float64_first_batch': float((O[:1].double() - ref).abs().max() / ref.abs().max()),
    }
    if cpu:
        qh, kh, vh = (x[0].cpu() for x in (Q, K, V))
        _, med, _, threads = _host_timed(torch, lambda: torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, scale=scale), 1, 3)
        res['cpu_baseline'] = {'value': flop / B / med / 1e12, 'unit': 'TFLOP/s', 'cores': threads, 'kind': 'torch_cpu_eager',
                               'sample': f'the {Hd} heads of one sample through torch scaled_dot_product_attention, fp32, {threads} threads, '
                                         f'median of 3: {med * 1e3:.0f} ms'}
    return res


def bench_embedding(torch, core, steps, warmup, cpu):
    """Embedding rows for a batch of word ids (the step that feeds the LSTM): V 5000 as in
    examples/stacked_rnn/rnn_utils.py, E 256 to match the LSTM configurations, 1 Mi ids."""
    V, E, n = 5000, 256, 1 << 20
    gen = torch.Generator(device='cpu').manual_seed(1234)
    table = torch.randn((V, E), generator=gen).cuda()
    ids = torch.randint(0, V, (n,), generator=gen).cuda()
    out = torch.empty((n, E), device='cuda')
    ms, wall = _events_ms(torch, lambda: core.embedding_gather(table, ids, out=out, check=False), steps, warmup)
    nbytes = 4.0 * n * E + 8.0 * n + 4.0 * V * E          # rows written once, ids and the table read once
    res = {
        'metric': 'embedding rows/s', 'value': n / ms * 1e3, 'unit': 'rows/s', 'ms_per_step': ms, 'dtype': 'f32',
        'config': {'workload': 'embedding gather feeding the LSTM (rnn_utils.py:81-90)', 'vocab': V, 'width': E, 'ids': n},
        'roofline': {'bound': 'hbm', 'achieved': nbytes / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                     'frac': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'traffic': MEASURED_TRAFFIC_BYTES.get('embedding_gather_pow2_kernel'),
                     'kernel': 'embedding_gather_pow2_kernel',
                     'algorithmic_bytes_per_launch': nbytes},
    }
    if cpu:
        t, i = table.cpu(), ids.cpu()
        t0 = time.perf_counter()
        _ = t[i]
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': n / dt, 'unit': 'rows/s', 'cores': torch.get_num_threads(), 'kind': 'port',
                               'sample': f'torch index_select of the same {n} ids on the host, {dt:.2f} s'}
    return res


def bench_softmax(torch, core, steps, warmup, cpu):
    """Row softmax of [65536, 1027] fp32 (1027: the widest row of the reference's test, test_softmax.cc:77-87; rows
    that are not 16-byte aligned), beside torch.softmax; every element read once and written once."""
    rows, cols = 65536, 1027
    gen = torch.Generator(device='cpu').manual_seed(1234)
    x = (torch.randn((rows, cols), generator=gen) * 4).cuda()
    y = torch.empty_like(x)
    ci = ctypes.c_int
    run = lambda: core._check(core.lib.ftk_online_softmax_f32(core._ptr(x), core._ptr(y), ci(rows), ci(cols), core._stream()))
    ms, _ = _events_ms(torch, run, steps, warmup)
    ms_t, _ = _events_ms(torch, lambda: torch.softmax(x, 1, out=y), steps, warmup)
    nbytes = 2.0 * rows * cols * 4
    res = {
        'metric': 'softmax rows/s', 'value': rows / ms * 1e3, 'unit': 'rows/s', 'ms_per_step': ms, 'dtype': 'f32',
        'config': {'workload': 'row softmax through (max, denominator) pairs (online_softmax_op.cu:14-36)', 'rows': rows, 'cols': cols},
        'roofline': {'bound': 'hbm', 'achieved': nbytes / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                     'frac': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'traffic': MEASURED_TRAFFIC_BYTES.get('softmax_rows_in_registers_kernel'),
                     'kernel': 'softmax_rows_in_registers_kernel<64, 32, false>', 'algorithmic_bytes_per_launch': nbytes},
        'torch_softmax': {'ms_per_step': ms_t, 'gbs': nbytes / ms_t / 1e6},
    }
    if cpu:
        from oracle import c_oracle
        n = rows
        xs = x[:n].cpu().numpy()
        t0 = time.perf_counter()
        c_oracle.online_softmax(xs)
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': n / dt, 'unit': 'rows/s', 'cores': 1, 'kind': 'port',
                               'sample': f'{n} rows through oracle/oracle.c in {dt:.2f} s'}
    return res


def _grid_torch_planes(torch, xs, ys, W, U, b, D, L, B, H):
    """The reference's schedule for the grid RNN on torch ops: per plane d+i+j one gather of the four operands
    and of the plane's weights, batched products, tanh, one scatter (regions/region8.h:61-310), with the index
    tensors built beforehand.  Level 0 of the padded array holds the first block's inputs, level d+1 block d's
    outputs; row/column 0 of every level is the zero border."""
    A = torch.zeros((D + 1, L + 1, L + 1, 2, B, H), device='cuda')
    A[0, 1:, 1:, 0] = xs[:, None]
    A[0, 1:, 1:, 1] = ys[None, :]
    flat = A.view(-1, B, H)
    at = lambda lvl, i, j, w: ((lvl * (L + 1) + i) * (L + 1) + j) * 2 + w
    planes = []
    for m in range(D + 2 * L - 2):
        pos = [(d, i, m - d - i) for d in range(D) for i in range(L) if 0 <= m - d - i < L]
        ix = lambda f: torch.tensor([f(d, i, j) for d, i, j in pos], device='cuda')
        planes.append((ix(lambda d, i, j: at(d, i + 1, j + 1, 0)), ix(lambda d, i, j: at(d, i + 1, j + 1, 1)),
                       ix(lambda d, i, j: at(d + 1, i, j + 1, 0)), ix(lambda d, i, j: at(d + 1, i + 1, j, 1)),
                       ix(lambda d, i, j: at(d + 1, i + 1, j + 1, 0)), ix(lambda d, i, j: at(d + 1, i + 1, j + 1, 1)),
                       ix(lambda d, i, j: d)))

    def run():
        for pxi, pyi, sxi, syi, oxi, oyi, dsel in planes:
            s = torch.cat([flat[sxi], flat[syi]], dim=2)
            su = torch.baddbmm(b[dsel], s, U[dsel])
            w = W[dsel]
            flat[oxi] = torch.tanh(torch.baddbmm(su, flat[pxi], w))
            flat[oyi] = torch.tanh(torch.baddbmm(su, flat[pyi], w))
    return run, A


def bench_grid_rnn(torch, core, steps, warmup, cpu, baselines=True):
    """The reference's grid benchmark shape (stacked_grid_rnn.cu:108-118, run.sh:7: batch 32, depth 32, hidden 256,
    both lengths 10; shared parameters, a bias row per batch row), fp32, one launch per plane."""
    D, L, B, H = 32, 10, 32, 256
    gen = torch.Generator(device='cpu').manual_seed(1234)
    u = lambda *shape, s=1.0: ((torch.rand(shape, generator=gen) * 2 - 1) * s).cuda()
    sc = 2.0 / (3 * H) ** 0.5
    xs, ys = u(L, B, H), u(L, B, H)
    W, U, b = u(D, H, H, s=sc), u(D, 2 * H, H, s=sc), u(D, B, H, s=0.2)
    out = torch.empty((D, L, L, 2, B, H), device='cuda')
    ci = ctypes.c_int
    ws = torch.empty(core.lib.ftk_grid_rnn_workspace_bytes(D, H) // 2, dtype=torch.uint8, device='cuda')   # shared parameters: one direction's worth
    run = lambda: core._check(core.lib.ftk_grid_rnn_f32(
        core._ptr(xs), core._ptr(ys), core._ptr(W), core._ptr(U), core._ptr(b), core._ptr(W), core._ptr(U), core._ptr(b),
        core._ptr(out), ci(D), ci(L), ci(L), ci(B), ci(H), ci(B), ci(0), core._ptr(ws), ctypes.c_size_t(ws.numel()), core._stream()))
    ms, _ = _events_ms(torch, run, steps, warmup)
    if baselines:
        ms_plain, _ = _events_ms(torch, lambda: core.grid_rnn(xs, ys, W, U, b, W, U, b, out=out, relay_weights=False), steps, warmup)
        run()
        base, A = _grid_torch_planes(torch, xs, ys, W, U, b, D, L, B, H)
        ms_t, _ = _events_ms(torch, base, max(2, steps // 5), 1)
        err = (A[1:, 1:, 1:] - out).abs().max().item()
    npos = D * L * L
    # k per position: H of input per direction; H per neighbour that exists, once (shared parameters: the state
    # product serves both directions)
    ksum = sum(H * (2 + (i > 0) + (j > 0)) for i in range(L) for j in range(L)) * D
    flop = 2.0 * B * H * ksum
    res = {
        'metric': 'grid positions/s', 'value': npos / ms * 1e3, 'unit': 'positions/s', 'ms_per_step': ms, 'dtype': 'f32',
        'config': {'workload': 'stacked grid RNN forward (grid_lstm/stacked_grid_rnn.cu), one launch per plane d+i+j',
                   'depth': D, 'src_len': L, 'trg_len': L, 'batch': B, 'hidden': H, 'planes': D + 2 * L - 2},
        'roofline': {'bound': 'mfma', 'achieved': flop / ms / 1e9, 'peak': PEAK_F32_MATRIX_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': flop / ms / 1e9 / PEAK_F32_MATRIX_TFLOPS, 'traffic': MEASURED_TRAFFIC_BYTES.get('grid_rnn_plane_kernel_per_pass'),
                     'kernel': 'grid_rnn_plane_kernel<true, 8, true> (50 launches per pass, after two re-lay launches)',
                     'note': 'the whole forward (50 dependent launches) against the fp32 MFMA peak; planes near the '
                             'corners hold a handful of positions, so the chain of launches, not the matrix rate, bounds it'},
    }
    if baselines:
        res['torch_per_plane_gather_bmm_scatter'] = {'ms_per_step': ms_t, 'speedup': ms_t / ms, 'max_abs_diff': err}
        res['without_workspace'] = {'ms_per_step': ms_plain, 'note': 'parameters read where they lie, no re-laid copy'}
    if cpu:
        from oracle import kaleido_oracle as ko
        Dc = 2
        t0 = time.perf_counter()
        ref = ko.grid_rnn_batched(xs.cpu().numpy(), ys.cpu().numpy(), W[:Dc].cpu().numpy(), U[:Dc].cpu().numpy(), b[:Dc].cpu().numpy(),
                                  W[:Dc].cpu().numpy(), U[:Dc].cpu().numpy(), b[:Dc].cpu().numpy(), dtype=np.float32)
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': Dc * L * L / dt, 'unit': 'positions/s', 'cores': 1, 'kind': 'port',
                               'sample': f'the first {Dc} blocks ({Dc * L * L} positions) through the numpy oracle in {dt:.2f} s',
                               'max_abs_diff_vs_gpu': float(np.abs(ref - out[:Dc].cpu().numpy()).max())}
    return res


def bench_windowed_attention(torch, core, steps, warmup, cpu):
    """The reference's sparse-attention shape (examples/sparse_attention/sparse_attention.py:125-141: 16 heads of 64,
    window 5, dilation 2, three random positions, the commented sequence length 4096) at batch 16, fp32: Q, K, V read
    once, O written once."""
    G, S, D, W, dl, R = 256, 4096, 64, 5, 2, 3
    gen = torch.Generator(device='cpu').manual_seed(1234)
    Q, K, V = ((torch.randn((G, S, D), generator=gen) * (2.0 / D ** 0.5 if i == 0 else 1.0)).cuda() for i in range(3))
    extra = torch.randint(0, S, (G, S, R), generator=gen, dtype=torch.int32).cuda()
    O = torch.empty_like(Q)
    ci = ctypes.c_int
    run = lambda: core._check(core.lib.ftk_windowed_attn_f32(core._ptr(Q), core._ptr(K), core._ptr(V), core._ptr(extra), core._ptr(O),
                                                             ci(G), ci(S), ci(D), ci(W), ci(dl), ci(R), ctypes.c_float(1.0), core._stream()))
    ms, _ = _events_ms(torch, run, steps, warmup)
    nbytes = 4.0 * G * S * D * 4 + G * S * R * 4
    res = {
        'metric': 'tokens/s (windowed attention)', 'value': G * S / ms * 1e3, 'unit': 'tokens/s', 'ms_per_step': ms, 'dtype': 'f32',
        'config': {'workload': 'windowed + random attention (shifted_slide + sparse_attn, sparse_attention.py:25-71)', 'batch_x_heads': G,
                   'seq_len': S, 'head_dim': D, 'window': W, 'dilation': dl, 'random': R},
        'roofline': {'bound': 'hbm', 'achieved': nbytes / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                     'frac': nbytes / ms / 1e6 / PEAK_HBM_GBS, 'traffic': MEASURED_TRAFFIC_BYTES.get('windowed_attn_kernel'),
                     'kernel': 'windowed_attn_kernel<16, 1>', 'algorithmic_bytes_per_launch': nbytes},
    }
    if cpu:
        from oracle import kaleido_oracle as ko
        n = 2
        t0 = time.perf_counter()
        ref = ko.windowed_attention(Q[:n].cpu().numpy(), K[:n].cpu().numpy(), V[:n].cpu().numpy(), W, dl, extra[:n].cpu().numpy(), dtype=np.float32)
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': n * S / dt, 'unit': 'tokens/s', 'cores': 1, 'kind': 'port',
                               'sample': f'{n} of {G} sequences ({n * S} tokens) through the numpy oracle in {dt:.2f} s',
                               'max_abs_diff_vs_gpu': float(np.abs(ref - O[:n].cpu().numpy()).max())}
    return res


def bench_gemm(torch, core, steps, warmup, cpu):
    """The plain fp16 product (ftk_gemm_f16) on its own: 8192^3, beside torch.mm."""
    M = N = K = 8192
    gen = torch.Generator(device='cpu').manual_seed(1234)
    A = (torch.randn((M, K), generator=gen) / K ** 0.5).half().cuda()
    B = torch.randn((K, N), generator=gen).half().cuda()
    C = torch.empty((M, N), dtype=torch.float16, device='cuda')
    ms, _ = _events_ms(torch, lambda: core.gemm(A, B, out=C), steps, warmup)
    ref = C.clone()
    ms_t, _ = _events_ms(torch, lambda: torch.mm(A, B, out=C), steps, warmup)
    flop = 2.0 * M * N * K
    res = {
        'metric': 'TFLOP/s (plain GEMM)', 'value': flop / ms / 1e9, 'unit': 'TFLOP/s', 'ms_per_step': ms, 'dtype': 'f16',
        'config': {'workload': 'plain GEMM building block (ftk_gemm_f16), row-major A, B, C', 'M': M, 'N': N, 'K': K, 'accumulate': 'f32'},
        'roofline': {'bound': 'mfma', 'achieved': flop / ms / 1e9, 'peak': PEAK_F16_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': flop / ms / 1e9 / PEAK_F16_TFLOPS, 'traffic': MEASURED_TRAFFIC_BYTES.get('gemm_8192'),
                     'kernel': 'gemm_f16_tile_kernel'},
        'torch_mm': {'ms_per_step': ms_t, 'tflops': flop / ms_t / 1e9,
                     'max_rel_diff': float((C.float() - ref.float()).abs().max() / ref.float().abs().max())},
    }
    if cpu:
        n = 1024
        a, b = A[:n, :n].float().cpu(), B[:n, :n].float().cpu()
        t0 = time.perf_counter()
        _ = a @ b
        dt = time.perf_counter() - t0
        res['cpu_baseline'] = {'value': 2.0 * n ** 3 / dt / 1e12, 'unit': 'TFLOP/s', 'cores': torch.get_num_threads(), 'kind': 'port',
                               'sample': f'torch fp32 matmul of a {n}^3 corner on the host, {dt:.3f} s'}
    return res


def _unfused_lstm_baseline(torch, core, xs, WU, hs, cs, dil=None):
    """Per-step GEMM (rocBLAS/hipBLASLt through torch) + one elementwise kernel, layer-major:
    the structure of benchmarks/rnn/fractaltensor/stacked_lstm (utils.h:559-625).  Returns a
    callable that replays the whole forward pass as one HIP graph, and the eager callable."""
    L, T, B, H = hs.shape
    W = WU[:, :H].contiguous()
    U = WU[:, H:].contiguous()
    xw = torch.empty((T * B, 4 * H), device='cuda')
    gates = torch.empty((B, 4 * H), device='cuda')

    def forward():
        inp = xs
        for l in range(L):
            d = 1 if dil is None else dil[l]
            torch.mm(inp.reshape(T * B, H), W[l], out=xw)        # x@W for all steps in one GEMM
            for t in range(T):
                g = xw[t * B:(t + 1) * B]
                if t >= d:
                    torch.addmm(g, hs[l, t - d], U[l], out=gates)  # per-step h@U
                    core.lstm_elementwise(gates, None, cs[l, t - d], out=(hs[l, t], cs[l, t]))
                else:
                    core.lstm_elementwise(g, None, None, out=(hs[l, t], cs[l, t]))
            inp = hs[l]

    forward()
    torch.cuda.synchronize()
    graph = None
    try:
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            forward()
        torch.cuda.current_stream().wait_stream(s)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            forward()
    except Exception as e:  # graph capture is an optimisation of the baseline, not a requirement
        print(f'# baseline graph capture unavailable: {e}', file=sys.stderr)
        graph = None
    return forward, graph


def bench_lstm(torch, core, steps, warmup, cpu, dilated, baselines=True):
    if dilated:
        L, T, B, H = 6, 128, 256, 256
        dil = [1, 2, 4, 8, 16, 32]
        name = 'dilated LSTM, BASELINE.json configs[4]'
    else:
        L, T, B, H = 32, 64, 256, 256
        dil = None
        name = 'stacked LSTM, BASELINE.json configs[3]'
    flop = 2.0 * L * T * B * (2 * H) * (4 * H)
    gen = torch.Generator(device='cpu').manual_seed(1234)
    xs = torch.randn((T, B, H), generator=gen).cuda()
    WU = ((torch.rand((L, 2 * H, 4 * H), generator=gen) - 0.5) / 8).cuda()   # U(-1/16, 1/16)
    hs = torch.empty((L, T, B, H), device='cuda')
    cs = torch.empty_like(hs)
    ws = torch.empty(core.stacked_lstm_workspace_bytes(L, T, B, H), dtype=torch.uint8, device='cuda')
    fused = lambda: core.stacked_lstm(xs, WU, dilations=dil, out=(hs, cs), workspace=ws)
    products = core.get_lstm_products()          # 'f16x3' unless FTK_LSTM_PRODUCTS says otherwise
    ms, wall = _events_ms(torch, fused, steps, warmup)
    status = core.persistent_status(ws)
    assert status == 0, 'the persistent launch drained early'
    small_states = core.stacked_lstm_small_states(ws)
    ref_h = hs.clone()
    executed = 3.0 * flop if products == 'f16x3' else flop      # MFMA flops the kernel issues
    peak = PEAK_F16_TFLOPS if products == 'f16x3' else PEAK_F32_MATRIX_TFLOPS
    extra = {}
    if baselines:
        # the same launch with the other way of forming the gate GEMM's products
        other = 'f32' if products == 'f16x3' else 'f16x3'
        core.set_lstm_products(other)
        ms_other, _ = _events_ms(torch, fused, max(2, steps // 2), 1)
        other_diff = float((hs - ref_h).abs().max() / ref_h.abs().max())
        core.set_lstm_products(products)
        # per-stage launches of the fused cell (no persistent kernel)
        ms_wave, _ = _events_ms(torch, lambda: core.stacked_lstm(xs, WU, dilations=dil, out=(hs, cs), schedule='wavefront'),
                                max(2, steps // 4), 1)
        # unfused GPU baseline
        hs_b = torch.empty_like(hs)
        cs_b = torch.empty_like(cs)
        eager, graph = _unfused_lstm_baseline(torch, core, xs, WU, hs_b, cs_b, dil)
        nb = max(2, steps // 4)
        ms_eager, _ = _events_ms(torch, eager, nb, 1)
        ms_graph = None
        if graph is not None:
            hs_b.zero_()
            ms_graph, _ = _events_ms(torch, graph.replay, nb, 2)
        base_err = float((hs_b - ref_h).abs().max() / ref_h.abs().max())
        assert base_err <= 1e-4 and other_diff <= 1e-4, f'fused stack differs from its baselines: {base_err:.3e}, {other_diff:.3e}'
        ms_base = ms_graph if ms_graph is not None else ms_eager
        # the same stack on a ragged batch: row lengths fall linearly from T to T/4 across the (sorted) batch
        lens = [max(1, T - (3 * T * b) // (4 * B)) for b in range(B)]
        active = [sum(1 for v in lens if v > t) for t in range(T)]
        ms_ragged, _ = _events_ms(torch, lambda: core.stacked_lstm(xs, WU, dilations=dil, out=(hs, cs), workspace=ws,
                                                                   active_rows=active), max(2, steps // 2), 1)
        live_blocks = sum((a + 31) // 32 for a in active) / float(T * ((B + 31) // 32))
        extra = {
            'ragged_batch': {'ms_per_step': ms_ragged, 'row_lengths': f'{lens[0]} .. {lens[-1]}, linear over the sorted batch',
                             'live_fraction_of_row_blocks': live_blocks, 'time_vs_dense': ms_ragged / ms},
            'other_products': {'products': other, 'ms_per_step': ms_other, 'sequences_per_s': B / ms_other * 1e3,
                               'max_rel_diff_vs_default': other_diff},
            'per_stage_launches': {'ms_per_step': ms_wave, 'sequences_per_s': B / ms_wave * 1e3},
            'unfused_gpu_baseline': {'ms_per_step_hip_graph': ms_graph, 'ms_per_step_eager': ms_eager,
                                     'sequences_per_s': B / ms_base * 1e3, 'speedup_of_fused': ms_base / ms,
                                     'speedup_of_fused_vs_eager': ms_eager / ms,
                                     'max_rel_diff_vs_fused': base_err,
                                     'what': 'one x@W GEMM per layer + per-step h@U GEMM (torch/rocBLAS) + one '
                                             'elementwise kernel per step, layer-major; speedup_of_fused is against '
                                             'the HIP-graph replay of that sequence (no launch overhead), '
                                             'speedup_of_fused_vs_eager against its eager launches'},
        }

    res = {
        'metric': 'stacked-LSTM sequences/s', 'value': B / ms * 1e3, 'unit': 'sequences/s', 'ms_per_step': ms,
        'dtype': 'f32 (gate products as three f16 MFMAs of split operands, f32 accumulate)' if products == 'f16x3' else 'f32',
        'config': {'workload': name, 'layers': L, 'batch': B, 'seq_len': T, 'hidden': H,
                   'dilations': dil, 'outputs': 'h and c of every layer at every step', 'products': products},
        'tflops': flop / ms / 1e9,
        'frac_of_f32_matrix_peak_algorithmic': flop / ms / 1e9 / PEAK_F32_MATRIX_TFLOPS,
        'persistent_status': status,
        # the roofline of the unit that executes: MFMA flops issued (three f16 MFMAs per fp32 product in f16x3 mode)
        # against the peak of that MFMA type.  The algorithmic flops (2*B*2H*4H per cell) against the fp32 matrix peak
        # are the named extra above; in f16x3 mode that ratio passes 1 and is no roofline fraction.
        'roofline': {'bound': 'mfma', 'achieved': executed / ms / 1e9, 'peak': peak, 'unit': 'TFLOP/s',
                     'frac': executed / ms / 1e9 / peak,
                     'what': 'MFMA flops issued (three f16 products per fp32 product in f16x3 mode) against the peak of '
                             'the MFMA type that executes them',
                     'algorithmic': {'tflops': flop / ms / 1e9, 'f32_matrix_peak': PEAK_F32_MATRIX_TFLOPS,
                                     'ratio_to_f32_matrix_peak': flop / ms / 1e9 / PEAK_F32_MATRIX_TFLOPS},
                     'traffic': MEASURED_TRAFFIC_BYTES.get('lstm_persistent_kernel' + ('_dilated' if dilated else '')),
                     'algorithmic_bytes_per_launch': 4.0 * (T * B * H + L * 2 * H * 4 * H + 2 * L * T * B * H),
                     'kernel': 'lstm_persistent_kernel'},
    }
    res.update(extra)
    if cpu:
        # the batched LSTM loop on torch CPU, the whole configuration: one [B, 2H] @ [2H, 4H] product and the gate
        # arithmetic as torch operators per layer and step
        xc, WUc = xs.cpu(), WU.cpu()
        out, med, best, threads = _host_timed(torch, lambda: _lstm_torch_cpu(torch, xc, WUc, dil), 1, 3)
        # the tolerance of the path: largest difference over the whole output (every layer's h) relative to its largest
        # value.  Beside it, per layer relative to that layer's own largest value: layers that fade towards zero
        # (config 4's upper ones: no bias, small weights) fall below what the fixed scale of the split products'
        # fp16 planes resolves, which the status block's small-states word reports (ftk_stacked_lstm_small_states)
        top = max(float(o.abs().max()) for o in out)
        per_layer = [(float((ref_h[l].cpu() - out[l]).abs().max()), float(out[l].abs().max())) for l in range(L)]
        diff = max(e for e, _ in per_layer) / top
        assert diff <= 1e-4, diff
        worst = max(range(L), key=lambda l: per_layer[l][0] / max(per_layer[l][1], 1e-300))
        layer_rel = {'worst_layer': worst, 'rel_to_that_layers_max': per_layer[worst][0] / max(per_layer[worst][1], 1e-300),
                     'that_layers_max_abs_h': per_layer[worst][1], 'top_layers_max_abs_h': per_layer[L - 1][1],
                     'small_states_word': small_states}
        res['cpu_baseline'] = {'value': B / med, 'unit': 'sequences/s', 'cores': threads, 'kind': 'torch_cpu_eager',
                               'sample': f'the whole configuration: per layer and step one [{B},{2 * H}] @ [{2 * H},{4 * H}] product '
                                         f'and the gate arithmetic as torch CPU operators (fp32), torch.set_num_threads({threads}) '
                                         f'of {os.cpu_count()} host CPUs, 1 warm-up + 3 timed runs, median {med:.2f} s (min {best:.2f} s)',
                               'ms_per_step': med * 1e3, 'max_rel_diff_vs_gpu': diff, 'per_layer_diff_vs_gpu': layer_rel,
                               'gpu_speedup': med * 1e3 / ms}
        # the per-sample operator program (scan over time of map over batch of [1,H] cells, four gate products per
        # cell: the reference's execution model) on a bounded sample, scaled by cells to the configuration
        from fractaltensor_amd import programs
        Ls, Ts, Bs = 2, 8, 32
        Wss, Uss, bss = programs.make_lstm_params(Ls, H, 1.0 / 16, 1234, bias=False)
        xss = programs.make_sequence_batch(Ts, Bs, H, 1234)
        prog = (lambda: programs.dilated_lstm(xss, Wss, Uss, bss)) if dilated else (lambda: programs.stacked_lstm(xss, Wss, Uss, bss))
        _, med_e, _, _ = _host_timed(torch, prog, 0, 2)
        full_seconds = med_e * (L * T * B) / (Ls * Ts * Bs)
        res['cpu_baseline']['eager_per_sample'] = {
            'value': B / full_seconds, 'unit': 'sequences/s',
            'sample': f'{Ls} layers x {Ts} steps x {Bs} samples of the eager operator program on torch CPU in {med_e:.2f} s, '
                      f'scaled by cells to the full configuration'}
        from oracle import c_oracle
        Ls, Ts, Bs = (2, 32, 256) if not dilated else (2, 32, 256)
        x = xs[:Ts, :Bs].cpu().numpy()
        w = WU[:Ls].cpu().numpy()
        t0 = time.perf_counter()
        c_oracle.stacked_lstm(x, w, None, None if dil is None else dil[:Ls])
        dt = time.perf_counter() - t0
        full_seconds = dt * (L * T * B) / (Ls * Ts * Bs)
        res['cpu_baseline']['scalar_c_port'] = {'value': B / full_seconds, 'unit': 'sequences/s', 'cores': 1,
                                                'sample': f'{Ls} layers x {Ts} steps x {Bs} rows through oracle/oracle.c in {dt:.1f} s, '
                                                          f'scaled by cell-rows to the full configuration'}
    return res


def bench_config1(torch, core, steps, warmup, cpu):
    """BASELINE.json configs[0]: one LSTM layer, B 64, T 16, H 256, fp32.  The reference runs this as its eager operator
    program on the host (examples/stacked_rnn/stacked_rnn.py:13-80); that program, written against this package's
    operators (fractaltensor_amd/programs.py), is the cpu_eager leg: per-sample [1,H] tensors, scan over time, map
    over batch, four gate products per cell, on torch CPU.  The batched leg is the same arithmetic as one
    [64,512] @ [512,1024] product per step, which separates operator dispatch from host GEMM speed."""
    from fractaltensor_amd import programs
    from fractaltensor_amd.kaleido.operations import fused
    L, T, B, H = 1, 16, 64, 256
    flop = 2.0 * L * T * B * (2 * H) * (4 * H)
    Wss, Uss, bss = programs.make_lstm_params(L, H, 0.1, 1234, bias=False)
    xss = programs.make_sequence_batch(T, B, H, 1234)
    xs = xss.as_dense().reshape(T, B, H).cuda()
    W, U = Wss.as_dense(), Uss.as_dense()                      # [L, 4, H, H]
    WU = torch.cat([W.permute(0, 2, 1, 3).reshape(L, H, 4 * H), U.permute(0, 2, 1, 3).reshape(L, H, 4 * H)], dim=1).contiguous()
    WUd = WU.cuda()
    hs = torch.empty((L, T, B, H), device='cuda')
    cs = torch.empty_like(hs)
    ws = torch.empty(core.stacked_lstm_workspace_bytes(L, T, B, H), dtype=torch.uint8, device='cuda')
    ms, wall = _events_ms(torch, lambda: core.stacked_lstm(xs, WUd, out=(hs, cs), workspace=ws), steps, warmup)
    core.stacked_lstm_check(ws)
    nbytes = 4.0 * (T * B * H + L * 2 * H * 4 * H + 2 * L * T * B * H)
    split = core.get_lstm_products() == 'f16x3'
    issued, peak = (3.0 * flop, PEAK_F16_TFLOPS) if split else (flop, PEAK_F32_MATRIX_TFLOPS)
    res = {
        'metric': 'stacked-LSTM sequences/s', 'value': B / ms * 1e3, 'unit': 'sequences/s', 'ms_per_step': ms,
        'dtype': 'f32 (gate products as three f16 MFMAs of split operands, f32 accumulate)' if split else 'f32',
        'config': {'workload': 'single-layer LSTM scan, BASELINE.json configs[0]', 'layers': L, 'batch': B, 'seq_len': T, 'hidden': H},
        'tflops': flop / ms / 1e9, 'host_wall_ms_per_step': wall,
        'frac_of_f32_matrix_peak_algorithmic': flop / ms / 1e9 / PEAK_F32_MATRIX_TFLOPS,
        'roofline': {'bound': 'mfma', 'achieved': issued / ms / 1e9, 'peak': peak, 'unit': 'TFLOP/s',
                     'frac': issued / ms / 1e9 / peak, 'traffic': None, 'kernel': 'lstm_persistent_kernel',
                     'what': 'MFMA flops issued (three f16 products per fp32 product in f16x3 mode) against the peak of '
                             'the MFMA type that executes them',
                     'note': '16 dependent steps of two row blocks on 8 of 256 compute units: a latency chain, not a throughput '
                             'shape', 'algorithmic_bytes_per_launch': nbytes},
    }
    if cpu:
        threads = _host_threads()
        before = torch.get_num_threads()
        torch.set_num_threads(threads)
        try:
            def timed(fn, warm, runs):
                for _ in range(warm):
                    out = fn()
                t = []
                for _ in range(runs):
                    t0 = time.perf_counter()
                    out = fn()
                    t.append(time.perf_counter() - t0)
                return out, sorted(t)[len(t) // 2], min(t)

            eager_out, eager_s, eager_min = timed(lambda: programs.stacked_lstm(xss, Wss, Uss, bss), 3, 10)
            xc, WUc = xs.cpu(), WU

            def batched():
                h = torch.zeros((B, H)); c = torch.zeros((B, H)); out = []
                for t in range(T):
                    g = torch.cat([xc[t], h], dim=1) @ WUc[0]
                    i, f, o, cand = g.chunk(4, 1)
                    c = torch.sigmoid(f) * c + torch.sigmoid(i) * torch.tanh(cand)
                    h = torch.sigmoid(o) * torch.tanh(c)
                    out.append(h)
                return torch.stack(out)

            batched_out, batched_s, batched_min = timed(batched, 3, 10)
        finally:
            torch.set_num_threads(before)
        eager_h = eager_out.as_dense().reshape(T, B, H)
        gpu_h = hs[L - 1].cpu()
        diff_eager = float((eager_h - gpu_h).abs().max() / gpu_h.abs().max())
        diff_batched = float((batched_out - gpu_h).abs().max() / gpu_h.abs().max())
        assert diff_eager <= 1e-4 and diff_batched <= 1e-4, (diff_eager, diff_batched)
        res['cpu_baseline'] = {
            'value': B / eager_s, 'unit': 'sequences/s', 'cores': threads, 'kind': 'torch_cpu_eager',
            'sample': f'the whole configuration: the eager operator program (programs.stacked_lstm: map over {B} samples of '
                      f'[1,{H}] tensors inside a scan over {T} steps, four gate products per cell) on torch CPU, '
                      f'torch.set_num_threads({threads}) of {os.cpu_count()} host CPUs, 3 warm-up + 10 timed runs, median '
                      f'{eager_s * 1e3:.1f} ms (min {eager_min * 1e3:.1f} ms)',
            'ms_per_step': eager_s * 1e3, 'max_rel_diff_vs_gpu': diff_eager,
            'batched': {'value': B / batched_s, 'unit': 'sequences/s', 'ms_per_step': batched_s * 1e3, 'min_ms': batched_min * 1e3,
                        'max_rel_diff_vs_gpu': diff_batched,
                        'what': f'the same layer as one [{B},{2 * H}] @ [{2 * H},{4 * H}] torch CPU product per step + torch '
                                f'gate arithmetic, {threads} threads, 3 warm-up + 10 timed runs, median'},
            'gpu_speedup_vs_eager': eager_s * 1e3 / ms, 'gpu_speedup_vs_batched': batched_s * 1e3 / ms,
        }
    return res


def bench_lstm_f16(torch, core, steps, warmup, cpu, H, baselines=True):
    """fp16-storage stack at the three hidden sizes of the reference's sweep (cute_stacked_lstm/stacked_lstm.cu:185-187):
    256 and 512 in the persistent kernel, 1024 through the streaming cell kernel, one launch per stage of cells."""
    L, T, B = 32, 64, 256
    flop = 2.0 * L * T * B * (2 * H) * (4 * H)
    gen = torch.Generator(device='cpu').manual_seed(1234)
    xs = torch.randn((T, B, H), generator=gen).half().cuda()
    WU = ((torch.rand((L, 2 * H, 4 * H), generator=gen) - 0.5) / {256: 8, 512: 12}.get(H, 16)).half().cuda()
    hs = torch.empty((L, T, B, H), dtype=torch.float16, device='cuda')
    cs = torch.empty_like(hs)
    ws = torch.empty(int(core.lib.ftk_stacked_lstm_f16_workspace_bytes(L, T, B, H)), dtype=torch.uint8, device='cuda')
    fused = lambda: core.stacked_lstm_f16(xs, WU, out=(hs, cs), workspace=ws)
    ms, wall = _events_ms(torch, fused, steps, warmup)
    on_chip = H == 256 or (H == 512 and L <= 16)   # deeper stacks of H = 512 are streamed like H = 1024 (the weights sit in the last-level cache)
    status = core.persistent_status(ws) if on_chip else None
    res = {
        'metric': 'stacked-LSTM sequences/s', 'value': B / ms * 1e3, 'unit': 'sequences/s', 'ms_per_step': ms, 'dtype': 'f16',
        'config': {'workload': f'stacked LSTM, fp16 storage, the H = {H} row of the reference sweep', 'layers': L, 'batch': B,
                   'seq_len': T, 'hidden': H, 'outputs': 'h and c of every layer at every step (fp16)', 'accumulate': 'f32'},
        'tflops': flop / ms / 1e9, 'persistent_status': status,
        'roofline': {'bound': 'mfma', 'achieved': flop / ms / 1e9, 'peak': PEAK_F16_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': flop / ms / 1e9 / PEAK_F16_TFLOPS,
                     'traffic': MEASURED_TRAFFIC_BYTES.get('lstm_persistent_kernel<2>' if H == 512 else 'lstm_persistent_kernel<3>'),
                     'kernel': 'lstm_persistent_kernel<2>' if H == 512 else 'lstm_persistent_kernel<3>'},
    }
    if not on_chip and H == 512:
        res['roofline']['kernel'] = 'lstm_cell_f16_kernel<true, 8, false>'
        res['roofline']['traffic'] = MEASURED_TRAFFIC_BYTES.get('lstm_cell_f16_kernel_h512_per_pass')
        res['config']['schedule'] = 'one launch of the streaming fp16 cell kernel per stage of independent cells'
    if not on_chip and H > 512:
        # every cell streams its layer's weights once (the stack's weights exceed the 256 MB of last-level cache), reads its
        # two input rows sets and c, writes h and c: the bytes that bound this schedule from below
        wbytes = L * T * (2 * H * 4 * H * 2.0)
        abytes = L * T * (5 * B * H * 2.0)
        res['roofline'] = {'bound': 'hbm', 'achieved': (wbytes + abytes) / ms / 1e6, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                           'frac': (wbytes + abytes) / ms / 1e6 / PEAK_HBM_GBS,
                           'traffic': MEASURED_TRAFFIC_BYTES.get('lstm_cell_f16_kernel_per_pass'),
                           'kernel': 'lstm_cell_f16_kernel<true, 8, false>',
                           'note': 'per launch: the cells of one stage; bytes = weights of every cell once + activations'}
        res['config']['schedule'] = 'one launch of the streaming fp16 cell kernel per stage of independent cells'
    if baselines:
        ref_h = hs.clone()
        W = WU[:, :H].contiguous()
        U = WU[:, H:].contiguous()
        hb = torch.empty_like(hs)

        def unfused():   # one x@W GEMM per layer, per step h@U (hipBLASLt through torch) and the state update as torch ops
            inp = xs
            for l in range(L):
                xw = torch.mm(inp.reshape(T * B, H), W[l]).reshape(T, B, 4 * H)
                h = None
                for t in range(T):
                    g = xw[t] if h is None else torch.addmm(xw[t], h, U[l])
                    i, f, o, c_ = g.chunk(4, 1)
                    c = torch.sigmoid(i) * torch.tanh(c_) if h is None else torch.sigmoid(f) * c + torch.sigmoid(i) * torch.tanh(c_)
                    h = torch.sigmoid(o) * torch.tanh(c)
                    hb[l, t] = h
                inp = hb[l]

        ms_eager, _ = _events_ms(torch, unfused, 2, 1)
        res['unfused_gpu_baseline'] = {'ms_per_step_eager': ms_eager, 'speedup_of_fused_vs_eager': ms_eager / ms,
                                       'max_rel_diff_vs_fused': float((hb.float() - ref_h.float()).abs().max() / ref_h.float().abs().max()),
                                       'what': 'torch fp16: one x@W GEMM per layer, per-step h@U GEMM, state update as torch ops, eager launches'}
    if cpu:
        from oracle import kaleido_oracle as ko
        Ls, Ts, Bs = 4, 64, 64
        t0 = time.perf_counter()
        ko.stacked_lstm_f16(xs[:Ts, :Bs].cpu().numpy(), WU[:Ls].cpu().numpy())
        dt = time.perf_counter() - t0
        full_seconds = dt * (L * T * B) / (Ls * Ts * Bs)
        res['cpu_baseline'] = {'value': B / full_seconds, 'unit': 'sequences/s', 'cores': 1, 'kind': 'port',
                               'sample': f'{Ls} layer x {Ts} steps x {Bs} rows through oracle/kaleido_oracle.py (numpy float64) in '
                                         f'{dt:.1f} s, scaled by cell-rows to the full configuration'}
    return res


def bench_lstm_f32_streamed(torch, core, steps, warmup, cpu, H):
    """The fp32 stack at the larger hidden sizes of the reference's sweep: weights streamed, one launch per stage of
    cells; split products through the fp16-MFMA streaming kernel (default) beside fp32 MFMAs."""
    L, T, B = 32, 64, 256
    flop = 2.0 * L * T * B * (2 * H) * (4 * H)
    gen = torch.Generator(device='cpu').manual_seed(1234)
    xs = torch.randn((T, B, H), generator=gen).cuda()
    WU = ((torch.rand((L, 2 * H, 4 * H), generator=gen) - 0.5) / (H ** 0.5 / 2)).cuda()
    hs = torch.empty((L, T, B, H), device='cuda')
    cs = torch.empty_like(hs)
    ws = torch.empty(int(core.stacked_lstm_workspace_bytes(L, T, B, H)), dtype=torch.uint8, device='cuda')
    run = lambda: core.stacked_lstm(xs, WU, out=(hs, cs), workspace=ws)
    before = core.get_lstm_products()
    try:
        core.set_lstm_products('f16x3')
        ms, _ = _events_ms(torch, run, steps, warmup)
        ref = hs.clone()
        core.set_lstm_products('f32')
        ms32, _ = _events_ms(torch, run, max(2, steps // 2), 1)
        diff = float((hs - ref).abs().max() / ref.abs().max())
    finally:
        core.set_lstm_products(before)
    res = {
        'metric': 'stacked-LSTM sequences/s', 'value': B / ms * 1e3, 'unit': 'sequences/s', 'ms_per_step': ms,
        'dtype': 'f32 (gate products as three f16 MFMAs of split operands, f32 accumulate)',
        'config': {'workload': f'stacked LSTM, fp32, the H = {H} row of the reference sweep', 'layers': L, 'batch': B, 'seq_len': T,
                   'hidden': H, 'outputs': 'h and c of every layer at every step',
                   'schedule': 'one launch of the split-product streaming cell kernel per stage of independent cells'},
        'tflops': flop / ms / 1e9, 'frac_of_f32_matrix_peak_algorithmic': flop / ms / 1e9 / PEAK_F32_MATRIX_TFLOPS,
        'fp32_mfma_products': {'ms_per_step': ms32, 'speedup_of_split_products': ms32 / ms, 'max_rel_diff': diff},
        'roofline': {'bound': 'mfma', 'achieved': 3 * flop / ms / 1e9, 'peak': PEAK_F16_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': 3 * flop / ms / 1e9 / PEAK_F16_TFLOPS,
                     'traffic': MEASURED_TRAFFIC_BYTES.get(f'lstm_cell_split4_kernel_h{H}_per_pass'), 'kernel': 'lstm_cell_split4_kernel',
                     'note': 'executed f16 MFMA flops (three per algorithmic product) against the f16 MFMA peak'},
    }
    if cpu:
        from oracle import c_oracle
        Ls, Ts, Bs = 2, 16, 64
        t0 = time.perf_counter()
        c_oracle.stacked_lstm(xs[:Ts, :Bs].cpu().numpy(), WU[:Ls].cpu().numpy(), None, None)
        dt = time.perf_counter() - t0
        full_seconds = dt * (L * T * B) / (Ls * Ts * Bs)
        res['cpu_baseline'] = {'value': B / full_seconds, 'unit': 'sequences/s', 'cores': 1, 'kind': 'port',
                               'sample': f'{Ls} layers x {Ts} steps x {Bs} rows through oracle/oracle.c in {dt:.1f} s, '
                                         f'scaled by cell-rows to the full configuration'}
    return res


def _under_profiler():
    """True when this process runs under a profiler's preloaded library (rocprofv3 sets these): a child process would
    inherit the preload, so no probe is spawned then."""
    pre = os.environ.get('LD_PRELOAD', '')
    return 'rocprof' in pre or any(k.startswith(('ROCPROF', 'ROCP_TOOL', 'ROCPROFILER')) for k in os.environ)


def probe_mfma_rate():
    """What the matrix pipes deliver under load: runs the stand-alone probe bench_probes/mfma_rate (built by
    `make -C bench_probes` / __graft_entry__.build()) as a child process and reports the fp16 MFMA rate it holds on
    random operands, the figure the fractions of the nominal peak on the other lines have to be read against."""
    import re
    import subprocess
    exe = os.path.join(ROOT, 'bench_probes', 'mfma_rate')
    if not os.path.exists(exe):
        raise SystemExit('bench.py --workload mfma_rate: bench_probes/mfma_rate is not built (make -C bench_probes)')
    if _under_profiler():
        raise SystemExit('bench.py: the MFMA-rate probe is a child process and is not started under a profiler')
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120, check=True).stdout
    alone = {}
    for ln in out.splitlines():
        m = re.match(r'mfma alone, (.+?)\s+([\d.]+) ns per MFMA\s+([\d.]+) clocks per MFMA\s+([\d.]+) GHz\s+->\s+(\d+) TFLOP/s', ln)
        if m:
            alone[m.group(1).strip()] = {'ns_per_mfma': float(m.group(2)), 'clocks_per_mfma': float(m.group(3)),
                                         'ghz': float(m.group(4)), 'tflops': float(m.group(5))}
    real = alone['random operands, 8 x 4 in turn']
    return {'metric': 'fp16 MFMA rate held on random operands (register-only v_mfma_f32_32x32x16_f16, one wave per SIMD)',
            'value': real['tflops'], 'unit': 'TFLOP/s', 'n_gpus': 1, 'steps': 3, 'warmup': 1, 'ms_per_step': 4000 * 32 * real['ns_per_mfma'] * 1e-6,
            'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f16', 'data': 'synthetic',
            'config': {'workload': 'matrix-pipe probe: 4000 x 32 MFMAs per wave, 1024 waves'},
            'roofline': {'bound': 'mfma', 'achieved': real['tflops'], 'peak': 2500.0, 'unit': 'TFLOP/s', 'frac': real['tflops'] / 2500.0, 'traffic': None},
            'cpu_baseline': None, 'mfma_alone': alone}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='b2b', choices=['b2b', 'config1', 'attention', 'stacked_lstm', 'dilated_lstm', 'lstm_f16_h256', 'lstm_f16_h512', 'lstm_f16_h1024', 'lstm_f32_h512', 'lstm_f32_h1024', 'attention_f32', 'attention_few_queries', 'gemm', 'online_softmax', 'embedding', 'grid_rnn', 'windowed_attention', 'b2b_ref_shapes', 'copy', 'mfma_rate'])
    ap.add_argument('--no-extras', action='store_true', help='measure only the chosen workload')
    ap.add_argument('--all', action='store_true', help='also the workloads either side of the path (fp16 / larger stacks, GEMM, softmax, embedding, grid RNN, windowed attention)')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--no-probe', action='store_true', help='do not start the stand-alone MFMA-rate probe (a child process) before the run')
    ap.add_argument('--no-baselines', action='store_true',
                    help='LSTM and grid workloads: only the fused kernel (no unfused GPU baseline, per-stage launches, other product mode, path without workspace)')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: every workload here is a single-device kernel '
              '(independent problems / heads / batch rows; no collectives). Run with --gpus 1.', file=sys.stderr)
        sys.exit(2)

    if args.workload == 'mfma_rate':
        print(json.dumps(probe_mfma_rate()))
        return
    # what the matrix pipes hold on random operands, measured by the stand-alone probe before this process touches
    # the GPU: the figure the fractions of the nominal MFMA peak below have to be read against
    held = None
    if not args.no_extras and not args.no_probe:
        try:
            pr = probe_mfma_rate()
            held = {'tflops_random_operands': pr['value'], 'frac_of_nominal_peak': pr['roofline']['frac'],
                    'tflops_constant_operands': pr['mfma_alone'].get('every lane the same constant', {}).get('tflops'),
                    'how': 'bench_probes/mfma_rate: register-only v_mfma_f32_32x32x16_f16, one wave per SIMD, 2.5 ms per run'}
        except (SystemExit, Exception) as e:   # the probe is an extra: its absence must not take the headline down
            held = {'error': repr(e)}

    import torch
    import fractaltensor_amd._core as core   # raises if libftkernels.so is missing: no fallback
    if not torch.cuda.is_available():
        print('bench.py needs a GPU', file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    cpu = not args.no_cpu

    runners = {
        'b2b': lambda s, w, c: bench_b2b(torch, core, s, w, c),
        'config1': lambda s, w, c: bench_config1(torch, core, s, w, c),
        'attention': lambda s, w, c: bench_attention(torch, core, s, w, c),
        'stacked_lstm': lambda s, w, c: bench_lstm(torch, core, max(3, s // 5), max(1, w // 5), c, False, not args.no_baselines),
        'dilated_lstm': lambda s, w, c: bench_lstm(torch, core, max(3, s // 5), max(1, w // 5), c, True, not args.no_baselines),
        'lstm_f16_h256': lambda s, w, c: bench_lstm_f16(torch, core, max(3, s // 5), max(1, w // 5), c, 256, not args.no_baselines),
        'lstm_f16_h512': lambda s, w, c: bench_lstm_f16(torch, core, max(3, s // 5), max(1, w // 5), c, 512, not args.no_baselines),
        'lstm_f16_h1024': lambda s, w, c: bench_lstm_f16(torch, core, max(3, s // 5), max(1, w // 5), c, 1024, not args.no_baselines),
        'lstm_f32_h512': lambda s, w, c: bench_lstm_f32_streamed(torch, core, max(3, s // 5), max(1, w // 5), c, 512),
        'lstm_f32_h1024': lambda s, w, c: bench_lstm_f32_streamed(torch, core, max(3, s // 10), 1, c, 1024),
        'b2b_ref_shapes': lambda s, w, c: bench_b2b_reference_shapes(torch, core, s, w, c),
        'attention_f32': lambda s, w, c: bench_attention_f32(torch, core, max(5, s // 2), max(2, w // 2), c),
        'attention_few_queries': lambda s, w, c: bench_attention_few_queries(torch, core, s, w, c),
        'gemm': lambda s, w, c: bench_gemm(torch, core, max(5, s // 5), max(2, w // 5), c),
        'online_softmax': lambda s, w, c: bench_softmax(torch, core, s, w, c),
        'embedding': lambda s, w, c: bench_embedding(torch, core, s, w, c),
        'grid_rnn': lambda s, w, c: bench_grid_rnn(torch, core, max(5, s // 2), max(2, w // 2), c, not args.no_baselines),
        'windowed_attention': lambda s, w, c: bench_windowed_attention(torch, core, s, w, c),
    }
    if args.workload == 'copy':
        runners = {'copy': lambda s, w, c: bench_copy(torch, core, s, w, c)}
        args.no_extras = True
    res = runners[args.workload](args.steps, args.warmup, cpu)
    line = {
        'metric': res.pop('metric'), 'value': res.pop('value'), 'unit': res.pop('unit'),
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': res.pop('ms_per_step'),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': res.pop('dtype'), 'data': 'synthetic', 'config': res.pop('config'),
        'roofline': res.pop('roofline'), 'cpu_baseline': res.pop('cpu_baseline', None),
    }
    line.update(res)
    info = core.device_info()
    line['device'] = {'arch': info.arch.decode(), 'compute_units': info.compute_units,
                      'host_cpus': os.cpu_count(), 'host_threads_used': _host_threads(), 'torch': torch.__version__}
    others = {}
    if not args.no_extras:
        # the other BASELINE.json configurations by default; the workloads either side of the path with --all
        extra_names = [n for n in runners if n != args.workload and (args.all or n in CONFIG_OF)]
        for name in extra_names:
            try:
                others[name] = runners[name](max(5, args.steps // 2), max(2, args.warmup // 2), cpu)
            except Exception as e:   # an extra must not take the headline down with it
                others[name] = {'error': repr(e)}
        line['other_workloads'] = others
    for r in [line] + [o for o in others.values() if 'roofline' in o]:
        if r['roofline'].get('traffic') is not None:
            r['roofline']['traffic_source'] = 'profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, not this run)'
    # one compact row per BASELINE.json configuration, last on the line so that a truncated record keeps it
    rows = {}
    for name, r in [(args.workload, line)] + list(others.items()):
        if name not in CONFIG_OF:
            continue
        if 'error' in r:
            rows[CONFIG_OF[name]] = {'workload': name, 'error': r['error']}
            continue
        diffs = [v for v in (r.get('cpu_baseline') or {}, r.get('unfused_gpu_baseline') or {})]
        diff = next((d[k] for d in diffs for k in ('max_rel_diff_vs_gpu', 'max_rel_diff_vs_fused') if k in d), None)
        sig = lambda v: None if v is None else float(f'{v:.4g}')   # four significant digits: the summary has to stay short
        rows[CONFIG_OF[name]] = {'workload': name, 'ms_per_step': sig(r['ms_per_step']), 'value': sig(r.get('value')), 'unit': r.get('unit'),
                                 'bound': r['roofline']['bound'], 'frac': sig(r['roofline']['frac']), 'max_rel_diff': sig(diff),
                                 'cpu_baseline': sig((r.get('cpu_baseline') or {}).get('value'))}
    if held is not None:
        line['fp16_mfma_rate_held'] = held
    line['configs'] = dict(sorted(rows.items()))
    print(json.dumps(line))


if __name__ == '__main__':
    main()
