#!/usr/bin/env python3
"""Benchmark of the Scatterbrain-local attention forward on one MI355X.

One "step" is one forward of BASELINE config 1 (fp32, B=2, H=1, L=3136, d=64, band 256 each side,
128 orthogonal-Gaussian random features) through the C ABI (flyhip_sblocal_forward: the key-side
pass, the fused band kernel, and the kernel that merges its partial results and adds the low-rank
term), inputs resident in HBM.  Prints ONE JSON line: tokens/s for the whole forward, the roofline of the dominant kernel
(the fused band kernel, timed with events on its stream inside the timed region), the CPU oracle
timed on this box's host cores, and -- as `extra` -- the block-sparse SDD / softmax / DSD stages
of BASELINE config 2 (bf16, B=8, H=12, L=4096, d=64, block 32) and whole-forward timings of
configs 3, 4 and 5.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# HBM bytes one launch of the dominant kernel moves at the benchmarked workload: rocprofv3 FETCH_SIZE / WRITE_SIZE
# readings scaled by a plain copy of known size, kept with the profile summaries they come from
TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'sblocal_fwd_config1_fp32_traffic.json')


def band_kernel_traffic():
    """Scaled read + write bytes per launch of the band kernel from the committed counter summary, or None."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
        return float(t['band_kernel']['hbm_read_bytes']) + float(t['band_kernel']['hbm_write_bytes'])
    except (OSError, KeyError, ValueError):
        return None


def band_kernel_pipe_view(kernel_ms):
    """The band kernel against the pipe it issues on: executed bf16 MFMA FLOPs per launch (counter
    SQ_INSTS_VALU_MFMA_MOPS_BF16 x 512, from the committed summary) over the live kernel time against the bf16 MFMA
    peak, and the share of the launch's SIMD cycles the matrix pipe was busy (SQ_VALU_MFMA_BUSY_CYCLES over
    1024 SIMDs x the kernel time the counters were taken at x the shader clock of that run)."""
    try:
        with open(TRAFFIC_FILE) as f:
            m = json.load(f)['band_kernel']['mfma']
        executed = float(m['mops_bf16']) * 512.0
        view = {'mfma_pipe': 'bf16', 'executed_flops_per_launch': executed, 'pipe_peak': PEAK_BF16_MFMA_TFLOPS,
                'pipe_frac': executed / (kernel_ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS,
                'mfma_busy_share': float(m['busy_cycles']) / (1024.0 * float(m['kernel_us']) * float(m['clock_mhz']))}
        return view
    except (OSError, KeyError, ValueError):
        return {'mfma_pipe': 'bf16', 'executed_flops_per_launch': None, 'pipe_peak': PEAK_BF16_MFMA_TFLOPS,
                'pipe_frac': None, 'mfma_busy_share': None}


def sblocal_flops(B, H, T, S, E, D, m, lc):
    """Algorithmic FLOPs of one forward (band pairs x 2(E+m+D), the two projections, K'^T V,
    Q'(K'^T V) and the normaliser dot) and the share of them the fused band kernel computes when
    the band of a query tile is split over several workgroups (the configuration benchmarked)."""
    lo, hi = lc // 2, (lc + 1) // 2
    pairs = B * H * sum(max(0, min(S, i + hi) - max(0, i - lo)) for i in range(T))
    band = pairs * 2 * (E + m + D)
    proj_q = 2 * B * H * T * E * (m // 2)
    proj_k = 2 * B * H * S * E * (m // 2)
    kv = 2 * B * H * S * m * D
    qkv = 2 * B * H * T * m * D + 2 * B * H * T * m
    total = band + proj_q + proj_k + kv + qkv
    fused = band                           # what the fused band kernel computes when the band of a query tile
    return total, fused                    # is split: projections in the key pass, low-rank term in the merge


def bench_sblocal(steps, warmup, cpu_baseline=True):
    import fly_amd
    from fly_amd import _lib
    from fly_amd.sblocal_attention import SBLocalPlan
    dev = torch.device('cuda:0')
    B, H, L, E, D, mh, lc = 2, 1, 3136, 64, 64, 64, 512
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, L, H, E, generator=g) * E ** -0.25 for _ in range(3))      # q, k, v ~ N(0,1) d^-1/4
    torch.manual_seed(0)
    P = fly_amd.gaussian_orthogonal_random_matrix(mh, E)
    t = 1 / math.sqrt(E)
    qd, kd, vd, Pd = (x.to(dev) for x in (q, k, v, P))
    plan = SBLocalPlan(B, H, L, L, E, mh, mh, torch.float32, dev, lc)
    out = torch.empty(B, L, H, D, device=dev)
    ln = torch.empty(B, H, L, device=dev)

    # Warm-up: the counted steps, then the same step until 50 ms have passed -- the clocks need tens of
    # milliseconds of load to settle on a workload, and a count of a few 30 microsecond steps is over long before that.
    w0 = time.perf_counter()
    done = 0
    while done < warmup or time.perf_counter() - w0 < 0.05:
        plan.run(qd, kd, vd, Pd, None, lc, t, out, ln)
        done += 1
        if done % 64 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    warmup_ms = (time.perf_counter() - w0) * 1e3
    t0 = time.perf_counter()
    for _ in range(steps):
        plan.run(qd, kd, vd, Pd, None, lc, t, out, ln)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # The dominant kernel is timed live on steps of the same loop that follow the timed ones (so that `wall` carries
    # no timing hook): the library launches the band kernel of a sampled step with two events that take the launch's
    # own begin and end time stamps, on its stream.  16 samples at least, one step in four at most.
    n_samples = max(16, min(64, steps // 4))
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_samples)]
    for a, b in ev:                      # create the underlying hipEvent_t objects before use
        a.record(); b.record()
    torch.cuda.synchronize()
    for a, b in ev:
        for _ in range(3):
            plan.run(qd, kd, vd, Pd, None, lc, t, out, ln)
        _lib.call('flyhip_sb_time_next_fwd', a.cuda_event, b.cuda_event)
        plan.run(qd, kd, vd, Pd, None, lc, t, out, ln)
    torch.cuda.synchronize()
    fwd_ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)

    # the same forward through the drop-in module (reference signature sblocal_attention.py:43-44): argument
    # checks, cached scratch, two result tensors per call
    mod = fly_amd.SBLocalAttention(lc, dim_heads=E, nb_features=2 * mh).to(dev).eval()
    mod.feature_map.projection_matrix.copy_(Pd)
    mod.feature_map.freeze_projection()
    with torch.no_grad():
        for _ in range(max(warmup, 3)):
            mod(qd, kd, vd)
        torch.cuda.synchronize()
        n_mod = max(steps, 200)
        t1 = time.perf_counter()
        for _ in range(n_mod):
            mod(qd, kd, vd)
        torch.cuda.synchronize()
        module_ms = (time.perf_counter() - t1) / n_mod * 1e3

    total_flops, fwd_flops = sblocal_flops(B, H, L, L, E, D, 2 * mh, lc)
    ms_per_step = wall / steps * 1e3
    achieved = fwd_flops / (fwd_ms * 1e-3) / 1e12
    roofline = {'bound': 'mfma', 'kernel': 'sblocal_fwd_x3_kernel<64,64,128,split>',
                'achieved': achieved, 'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                'frac': achieved / PEAK_FP32_MFMA_TFLOPS, 'traffic': band_kernel_traffic(),
                'kernel_ms': fwd_ms, 'flops_per_launch': fwd_flops, 'launches_timed': len(ev),
                'arithmetic': 'fp32 inputs, outputs and accumulation; products on v_mfma_f32_16x16x32_bf16 from '
                              'operands split into bf16 pieces (scores 3 piece products, feature overlap 4 on '
                              'features rounded to 17 bits, P V 5 with V rounded to 16 bits).  achieved / peak / frac '
                              'price the ALGORITHMIC fp32 FLOPs against the fp32 MFMA peak; mfma_pipe .. pipe_frac '
                              'price the piece products actually issued against the peak of the pipe they run on'}
    roofline.update(band_kernel_pipe_view(fwd_ms))
    res = {
        'tokens_per_s': B * L / (wall / steps),
        'ms_per_step': ms_per_step,
        'warmup_ms': warmup_ms,
        'module_forward_ms': module_ms,
        'roofline': roofline,
        'parity': None,
        'flops_per_step': total_flops,
    }

    if not cpu_baseline:
        res['cpu_baseline'] = None
        return res
    # CPU baseline leg: the oracle (a port of the reference op sequence) on the host cores, bounded
    # to about 12 s of work.  Its float64 result also checks the output of the steps just timed.
    from oracle import sblocal as osb
    ref_out, ref_ln = osb.sblocal_attention(q.double(), k.double(), v.double(), P.double(), lc)
    res['parity'] = {
        'out_rel_err': float((out.cpu().double() - ref_out).abs().max() / ref_out.abs().max()),
        'log_norm_rel_err': float((ln.cpu().double().unsqueeze(-1) - ref_ln).abs().max() / ref_ln.abs().max())}
    host_cpus = os.cpu_count() or 1
    torch.set_num_threads(min(host_cpus, 16))          # the box's CPU share for one GPU is 16 cores
    osb.sblocal_attention(q, k, v, P, lc)
    n, t0 = 0, time.perf_counter()
    while True:
        osb.sblocal_attention(q, k, v, P, lc)
        n += 1
        el = time.perf_counter() - t0
        if el > 12.0:
            break
    res['cpu_baseline'] = {'value': B * L * n / el, 'unit': 'tokens/s', 'cores': torch.get_num_threads(),
                           'host_cpus': host_cpus, 'kind': 'port',
                           'sample': f'{n} full-size forwards of the same workload (fp32 oracle, {el:.1f} s, '
                                     f'{torch.get_num_threads()} threads of {host_cpus} host CPUs)'}
    return res


def bench_blocksparse(steps, warmup):
    """BASELINE config 2: SDD -> softmax -> DSD, bf16, B=8, H=12, L=4096, d=64, block 32."""
    from fly_amd import matmul, softmax, FlatBlockButterflySparsityConfig
    dev = torch.device('cuda:0')
    B, H, L, d, block = 8, 12, 4096, 64, 32
    nb = L // block
    r = torch.arange(nb)
    band = ((r.view(-1, 1) - r.view(1, -1)).abs() <= 4)
    lay = (FlatBlockButterflySparsityConfig(8, 2, block).make_layout(L) > 0) | band
    layout = lay.long().unsqueeze(0).repeat(H, 1, 1)
    nnz = int(layout.sum())
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, H, L, d, generator=g).bfloat16().to(dev) for _ in range(3))
    sdd = matmul(layout, block, 'sdd', trans_b=True)
    dsd = matmul(layout, block, 'dsd')
    sm = softmax(layout, block)
    out = {}

    def timeit(fn):
        t0 = time.perf_counter()                 # warm-up by time as well as by count (settled clocks)
        done = 0
        while done < warmup or time.perf_counter() - t0 < 0.05:
            fn()
            done += 1
            if done % 8 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        # median of three batches: one stall of the issuing thread (tens of milliseconds now and then on a shared
        # host) would otherwise land in a single stage's figure
        reps = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            reps.append(e0.elapsed_time(e1) / steps)
        return sorted(reps)[1]

    qk = sdd(q, k)
    flops = 2 * B * nnz * block * block * d
    sp_bytes = B * nnz * block * block * 2
    dense_bytes = B * H * L * d * 2
    ms = timeit(lambda: sdd(q, k))
    out['sdd'] = {'ms': ms, 'tflops': flops / ms / 1e9, 'gbs': (sp_bytes + 2 * dense_bytes) / ms / 1e6}
    ms = timeit(lambda: sm(qk, scale=0.125))
    out['softmax'] = {'ms': ms, 'gbs': 2 * sp_bytes / ms / 1e6}
    ms = timeit(lambda: dsd(qk, v))
    out['dsd'] = {'ms': ms, 'tflops': flops / ms / 1e9, 'gbs': (sp_bytes + 2 * dense_bytes) / ms / 1e6}
    for st in out.values():
        st['hbm_frac'] = st['gbs'] / PEAK_HBM_GBS
    # the three stages as separate launches, and the one-kernel form BlockSparseAttention.forward uses
    # when it needs no gradients, weights or attention mask (same inputs, same result)
    from fly_amd import fused_attention
    fused = fused_attention(layout, block)
    ms3 = timeit(lambda: dsd(sm(sdd(q, k), scale=0.125), v))
    ref = dsd(sm(sdd(q, k), scale=0.125), v).float()
    got = fused(q, k, v, 0.125).float()
    ms = timeit(lambda: fused(q, k, v, 0.125))
    out['three_stage_attention_ms'] = ms3
    # a training step of the same attention (the three ops are autograd functions; the gradients run
    # on the tiled SDD / DSD kernels, the transposed-DSD kernel and the one-pass softmax gradient)
    qg, kg, vg = (t.detach().clone().requires_grad_() for t in (q, k, v))
    go = torch.randn(B, H, L, d, generator=g).bfloat16().to(dev)

    def train_step():
        o = dsd(sm(sdd(qg, kg), scale=0.125), vg)
        o.backward(go)
        qg.grad = kg.grad = vg.grad = None
    out['three_stage_attention_fwd_bwd_ms'] = timeit(train_step)
    del qg, kg, vg, go

    # the same training step through BlockSparseAttention: forward on the one-kernel attention (it keeps
    # a log-denominator per row), backward = probabilities again, dV, fused score gradient, dQ, dK
    from fly_amd import BlockSparseAttention

    class Layout:
        def __init__(self):
            self.block = block

        def make_layout(self, seqlen):
            return layout
    mod = BlockSparseAttention(Layout(), attention_dropout=0.0, max_seq_length=L).to(dev)
    qm, km, vm = (t.detach().transpose(1, 2).contiguous().requires_grad_() for t in (q, k, v))      # (B, L, H, d)
    gm = torch.randn(B, L, H, d, generator=g).bfloat16().to(dev)

    def module_step():
        o, _ = mod(qm, km, vm)
        o.backward(gm)
        qm.grad = km.grad = vm.grad = None
    out['module_fwd_bwd_ms'] = timeit(module_step)
    # ... with a key-padding mask (every second batch entry 500 keys short): the one-kernel forward reads it, and so do
    # the two launches of the backward (blocksparse_attention.py:117-127,146-152)
    from fly_amd import LengthMask
    lens = torch.full((B,), L, dtype=torch.long)
    lens[1::2] = L - 500
    pad_mask = LengthMask(lens.to(dev), max_len=L)

    def module_masked_step():
        o, _ = mod(qm, km, vm, key_padding_mask=pad_mask)
        o.backward(gm)
        qm.grad = km.grad = vm.grad = None
    out['module_key_padding_fwd_bwd_ms'] = timeit(module_masked_step)
    # ... and with the constructor's default attention dropout of 0.1 (blocksparse_attention.py:31,160): the mask
    # is a hash formed inside the same kernels; `fuse = False` is the op-by-op chain with nn.Dropout on the
    # stored probabilities
    mod_drop = BlockSparseAttention(Layout(), max_seq_length=L).to(dev).train()

    def module_drop_step():
        o, _ = mod_drop(qm, km, vm)
        o.backward(gm)
        qm.grad = km.grad = vm.grad = None
    out['module_dropout_fwd_bwd_ms'] = timeit(module_drop_step)
    with torch.no_grad():
        out['module_dropout_fwd_ms'] = timeit(lambda: mod_drop(qm, km, vm))
    mod_drop.fuse = False
    out['module_dropout_op_by_op_fwd_bwd_ms'] = timeit(module_drop_step)
    del qm, km, vm, gm, mod, mod_drop
    out['fused_attention'] = {'ms': ms, 'tflops': 2 * flops / ms / 1e9, 'mfma_bf16_frac': 2 * flops / ms / 1e9 / 2500.0,
                              'speedup_over_three_stages': ms3 / ms,
                              'max_diff_vs_three_stages': float((got - ref).abs().max() / ref.abs().max())}
    # what a plain device copy of the sparse tensor reaches on this box (read + write bytes per second)
    dst = torch.empty_like(qk)
    ms = timeit(lambda: dst.copy_(qk))
    out['plain_copy_gbs'] = 2 * sp_bytes / ms / 1e6
    out['config'] = f'bf16 B={B} H={H} L={L} d={d} block={block} nnz/head={nnz // H}'
    return out


def sblocal_train_step(q, k, v, P, lc, temp):
    """A closure running one forward + backward of Scatterbrain-local attention with respect to q, k, v (with the
    per-shape scratch cache that the module SBLocalAttention keeps between its calls)."""
    import fly_amd
    from fly_amd.sblocal_attention import ScratchCache
    qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
    go = torch.randn_like(v)
    cache = ScratchCache()

    def run():
        o = fly_amd.sblocal_attention_fn(qg, kg, vg, P, lc, temp, None, cache=cache)
        o = o[0] if isinstance(o, tuple) else o
        o.backward(go)
        qg.grad = kg.grad = vg.grad = None
    return run


def bench_other_configs():
    """Timings of the remaining BASELINE configs (stream events around whole forwards):
    3 = the two Scatterbrain-local layers of T2T-ViT-t-14 at batch 64 (fp32), 4 = the two Pixelfly
    block-sparse linears of the Mixer-B channel MLP (bf16), 5 = long-sequence Scatterbrain-local (bf16)."""
    import fly_amd
    from fly_amd.sblocal_attention import SBLocalPlan
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    torch.manual_seed(0)
    out = {}

    def timeit(fn, n=10, w=2):
        # warm-up by time as well as by count: the clocks take tens of milliseconds of load to settle on a workload
        # (a 0.3 ms forward timed after two calls reads 15 - 20 % above its steady state)
        t0 = time.perf_counter()
        done = 0
        while done < w or time.perf_counter() - t0 < 0.05:
            fn()
            done += 1
            if done % 8 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        reps = []
        for _ in range(3):                      # median of three timed runs of n calls
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            reps.append(e0.elapsed_time(e1) / n)
        return sorted(reps)[1]

    for L, dim in ((3136, 147), (784, 576)):
        B, H, E, mh, lc = 64, 1, 64, 64, 256
        q, k, v = (torch.randn(B, L, H, E, generator=g).to(dev) for _ in range(3))
        P = fly_amd.gaussian_orthogonal_random_matrix(mh, E).to(dev)
        plan = SBLocalPlan(B, H, L, L, E, mh, mh, torch.float32, dev, lc)
        o = torch.empty(B, L, H, E, device=dev)
        ln = torch.empty(B, H, L, device=dev)
        ms = timeit(lambda: plan.run(q, k, v, P, None, lc, dim ** -0.5, o, ln))
        fl, _ = sblocal_flops(B, H, L, L, E, E, 2 * mh, lc)
        out[f'config3_sblocal_fp32_B64_L{L}'] = {'ms': ms, 'tflops': fl / ms / 1e9, 'tokens_per_s': B * L / ms * 1e3,
                                                 'mfma_fp32_frac': fl / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS,
                                                 'fwd_bwd_ms': timeit(sblocal_train_step(q, k, v, P, lc, dim ** -0.5), n=5)}
        del q, k, v, o, ln, plan

    # training step of the headline configuration: forward on the fused kernels, gradients of q, k, v
    # on the two passes of the backward band kernel
    B, H, L, E, mh, lc = 2, 1, 3136, 64, 64, 512
    q, k, v = (torch.randn(B, L, H, E, generator=g).to(dev) * E ** -0.25 for _ in range(3))
    P = fly_amd.gaussian_orthogonal_random_matrix(mh, E).to(dev)
    out['config1_sblocal_fp32_fwd_bwd_ms'] = timeit(sblocal_train_step(q, k, v, P, lc, None), n=10)
    del q, k, v

    # Scatterbrain on a block-sparse support at the first T2T layer's size (the sbbs-* attention configs:
    # block 32, three sliding-window blocks, 32 features; here with one global block row / column)
    class WindowPlusGlobal:
        def __init__(self, block):
            self.block = block

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            r = torch.arange(nb)
            lay = ((r.view(-1, 1) - r.view(1, -1)).abs() <= 1).long()
            lay[:, 0] = 1
            lay[0, :] = 1
            return lay.unsqueeze(0)
    B, L, E = 64, 3136, 64
    sbbs = fly_amd.SBBlockSparseAttention(WindowPlusGlobal(32), dim_heads=E, nb_features=32, max_seq_length=L).to(dev)
    q, k, v = (torch.randn(B, L, 1, E, generator=g).to(dev) * E ** -0.25 for _ in range(3))
    with torch.no_grad():
        out['sbblocksparse_fp32_B64_L3136_block32_m32'] = {'ms': timeit(lambda: sbbs(q, k, v), n=5)}
        # training-mode dropout of the exact weights inside the same kernels (a fresh seed per call)
        sbbs_drop = fly_amd.SBBlockSparseAttention(WindowPlusGlobal(32), dim_heads=E, nb_features=32, max_seq_length=L,
                                                   attention_dropout=0.1).to(dev).train()
        out['sbblocksparse_fp32_B64_L3136_block32_m32']['dropout_fwd_ms'] = timeit(lambda: sbbs_drop(q, k, v), n=5)
        del sbbs_drop
    # its training step: fused forward, backward kernels walking the layout's blocks; beside it the op-by-op path
    qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
    go = torch.randn_like(v)

    def sbbs_step():
        o, _ = sbbs(qg, kg, vg)
        o.backward(go)
        qg.grad = kg.grad = vg.grad = None
    out['sbblocksparse_fp32_B64_L3136_block32_m32']['fwd_bwd_ms'] = timeit(sbbs_step, n=5)
    sbbs.fuse = False
    out['sbblocksparse_fp32_B64_L3136_block32_m32']['fwd_bwd_op_by_op_ms'] = timeit(sbbs_step, n=3)
    del q, k, v, sbbs, qg, kg, vg, go
    # the second T2T layer's size with the reference's settings for it (sbbs-*.yaml: block 16, 16 features): forward
    # on the fused kernels (a wave per block-row, half-tile masks) and op by op
    L = 784
    sbbs = fly_amd.SBBlockSparseAttention(WindowPlusGlobal(16), dim_heads=E, nb_features=16, max_seq_length=L).to(dev)
    q, k, v = (torch.randn(B, L, 1, E, generator=g).to(dev) * E ** -0.25 for _ in range(3))
    with torch.no_grad():
        ms_f = timeit(lambda: sbbs(q, k, v), n=5)
        sbbs.fuse = False
        ms_o = timeit(lambda: sbbs(q, k, v), n=3)
    out['sbblocksparse_fp32_B64_L784_block16_m16'] = {'ms': ms_f, 'op_by_op_ms': ms_o}
    qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
    go = torch.randn_like(v)

    def sbbs16_step():
        o, _ = sbbs(qg, kg, vg)
        o.backward(go)
        qg.grad = kg.grad = vg.grad = None
    sbbs.fuse = True
    out['sbblocksparse_fp32_B64_L784_block16_m16']['fwd_bwd_ms'] = timeit(sbbs16_step, n=5)
    sbbs.fuse = False
    out['sbblocksparse_fp32_B64_L784_block16_m16']['fwd_bwd_op_by_op_ms'] = timeit(sbbs16_step, n=3)
    del qg, kg, vg, go
    del q, k, v, sbbs

    cfg = fly_amd.FlatBlockButterflySparsityConfig(8, 2, block=32)
    torch.manual_seed(0)
    fc1 = fly_amd.BlockSparseLinear(768, 3072, cfg, bias=False).to(dev).to(torch.bfloat16)
    fc2 = fly_amd.BlockSparseLinear(3072, 768, cfg, bias=False).to(dev).to(torch.bfloat16)
    x = torch.randn(256 * 196, 768, generator=g).bfloat16().to(dev)
    h = torch.randn(256 * 196, 3072, generator=g).bfloat16().to(dev)
    w = torch.randn(3072, 768, generator=g).bfloat16().to(dev)
    with torch.no_grad():
        ms1, ms2 = timeit(lambda: fc1(x)), timeit(lambda: fc2(h))
        msd = timeit(lambda: torch.nn.functional.linear(x, w))
    fl = 2 * 50176 * 864 * 1024
    out['config4_pixelfly_linear_bf16'] = {
        'fc1_ms': ms1, 'fc1_tflops': fl / ms1 / 1e9, 'fc2_ms': ms2, 'fc2_tflops': fl / ms2 / 1e9,
        'fc1_hbm_gbs': (x.numel() + 50176 * 3072 + 864 * 1024) * 2 / ms1 / 1e6,
        'dense_library_gemm_768_3072_ms': msd}

    # one training step of the layer: forward, input gradient (DDS on untransposed blocks) and weight
    # gradient (split-K SDD), beside the same for a dense nn.Linear of the same shape
    def fwd_bwd(mod, inp):
        def run():
            y = mod(inp)
            y.backward(gy[: y.numel()].view_as(y))
            inp.grad = None
            for p_ in mod.parameters():
                p_.grad = None
        return run
    gy = torch.randn(50176 * 3072, generator=g).bfloat16().to(dev)
    xg, hg = x.clone().requires_grad_(), h.clone().requires_grad_()
    dense = torch.nn.Linear(768, 3072, bias=False).to(dev).to(torch.bfloat16)
    out['config4_pixelfly_linear_bf16'].update({
        'fc1_fwd_bwd_ms': timeit(fwd_bwd(fc1, xg), n=5), 'fc2_fwd_bwd_ms': timeit(fwd_bwd(fc2, hg), n=5),
        'dense_768_3072_fwd_bwd_ms': timeit(fwd_bwd(dense, xg), n=5)})
    del x, h, w, fc1, fc2, gy, xg, hg, dense

    B, L, H, E, mh, lc = 1, 16384, 16, 64, 128, 1024
    q, k, v = (torch.randn(B, L, H, E, generator=g) for _ in range(3))
    idx = torch.randperm(L, generator=g)[: L // 20]
    k[:, idx] *= 8
    q, k, v = (x.bfloat16().to(dev) for x in (q, k, v))
    P = fly_amd.gaussian_orthogonal_random_matrix(mh, E).to(dev)
    plan = SBLocalPlan(B, H, L, L, E, mh, mh, torch.bfloat16, dev, lc)
    o = torch.empty(B, L, H, E, device=dev, dtype=torch.bfloat16)
    ln = torch.empty(B, H, L, device=dev)
    ms = timeit(lambda: plan.run(q, k, v, P, None, lc, 0.125, o, ln))
    msk = timeit(lambda: plan.run_keys(q, k, v, P, None, 0.125))
    fl, band_fl = sblocal_flops(B, H, L, L, E, E, 2 * mh, lc)
    out['config5_sblocal_bf16_L16384'] = {'ms': ms, 'key_pass_ms': msk, 'tflops': fl / ms / 1e9,
                                          'tokens_per_s': B * L / ms * 1e3, 'mfma_bf16_frac': fl / ms / 1e9 / 2500.0}
    # plain local attention (LocalAttention, local_attention.py:50-92) on the same inputs: the band softmax alone
    from fly_amd.local_attention import local_forward
    pairs = band_fl / (2 * (E + 2 * mh + E))                 # band pairs, from the count above
    ms = timeit(lambda: local_forward(q, k, v, lc, softmax_temp=0.125))
    out['local_attention_bf16_L16384'] = {'ms': ms, 'tflops': pairs * 2 * (E + E) / ms / 1e9}
    from fly_amd.local_attention import local_attention_fn
    qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
    go = torch.randn(B, L, H, E, generator=g).bfloat16().to(dev)

    def local_step():
        local_attention_fn(qg, kg, vg, lc, softmax_temp=0.125).backward(go)
        qg.grad = kg.grad = vg.grad = None
    out['local_attention_bf16_L16384']['fwd_bwd_ms'] = timeit(local_step, n=5)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=2000)
    ap.add_argument('--warmup', type=int, default=50)
    ap.add_argument('--no-blocksparse', action='store_true', help='skip the config 2 stages')
    ap.add_argument('--no-other-configs', action='store_true', help='skip the timings of configs 3, 4, 5')
    ap.add_argument('--skip-cpu', action='store_true', help='skip the CPU baseline leg (profiling runs)')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run a plain 256 MiB device copy: its FETCH_SIZE / WRITE_SIZE readings '
                         'give the scale of the traffic counters')
    ap.add_argument('--train-step', choices=['config1', 'config3'], default=None,
                    help='profiling runs: only time --steps forward + backward steps of Scatterbrain-local attention at '
                         'that configuration (fp32; config3 = first T2T layer, B=64 L=3136 window 256) and print their time')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py: this build measures one GPU; --gpus must be 1 (nothing here shards over devices)',
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print('bench.py: no GPU visible', file=sys.stderr)
        sys.exit(1)
    if args.train_step:
        import fly_amd
        dev = torch.device('cuda:0')
        g = torch.Generator().manual_seed(0)
        torch.manual_seed(0)
        B, L, lc, temp, scale = (2, 3136, 512, None, 64 ** -0.25) if args.train_step == 'config1' else (64, 3136, 256, 147 ** -0.5, 1.0)
        q, k, v = (torch.randn(B, L, 1, 64, generator=g).to(dev) * scale for _ in range(3))
        P = fly_amd.gaussian_orthogonal_random_matrix(64, 64).to(dev)
        step = sblocal_train_step(q, k, v, P, lc, temp)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        print(json.dumps({'train_step': args.train_step, 'steps': args.steps,
                          'fwd_bwd_ms': (time.perf_counter() - t0) / args.steps * 1e3}))
        return
    if args.copy_calibration:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device='cuda:0').normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    sb = bench_sblocal(args.steps, args.warmup, cpu_baseline=not args.skip_cpu)
    line = {
        'metric': 'SBLocal attention forward tokens/s (fp32, L=3136, d=64)',
        'value': sb['tokens_per_s'], 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'warmup_ms': sb['warmup_ms'], 'ms_per_step': sb['ms_per_step'], 'higher_is_better': True,
        'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'BASELINE config 1 (configs[0]): SBLocal fwd fp32 B=2 H=1 L=3136 d=64 '
                               'local_context=512 nb_features=128, seeded orthogonal-Gaussian projection'},
        'module_forward_ms': sb['module_forward_ms'],
        'roofline': sb['roofline'], 'cpu_baseline': sb['cpu_baseline'],
        'gpu_over_cpu': sb['tokens_per_s'] / sb['cpu_baseline']['value'] if sb['cpu_baseline'] else None,
        'parity': sb['parity'],
    }
    extra = {}
    if not args.no_blocksparse:
        extra['blocksparse_config2'] = bench_blocksparse(min(20, max(5, args.steps // 10)), 3)
    if not args.no_other_configs:
        extra.update(bench_other_configs())
    if extra:
        line['extra'] = extra
    print(json.dumps(line))


if __name__ == '__main__':
    main()
