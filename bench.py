"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline workload (the configuration the metric is quoted on): W8A16 decode GEMV at the LLaMA-7B MLP up-proj
shape, a f16 [1, 4096] x w int8 [4096, 11008] with per-column f16 scales.  One step = one pass over a ring of
RING distinct weight matrices (RING * 45 MB > 2 x the 256 MB last-level cache), so every launch streams its
weights from DRAM.  A step is captured once into a HIP graph and replayed; `value` is algorithmic bytes per
step / wall time per step with all inputs resident in HBM.

The same JSON line carries
  roofline      the GEMV kernel's own duration (begin/end of the dispatch, HIP events armed through the
                library's timing hook, one launch at a time after the timed region) against 8 TB/s;
  cpu_baseline  the restated CPU route of the reference (oracle/cpu_baseline.c) on the host cores, on a
                bounded sample of the same workload;
  prefill       the M = 2048 GEMM of the same weight shape as TFLOP/s (second half of the metric);
  fp8_prefill   the e4m3 GEMM [4096, 8192] x [8192, 8192]^T -> bf16 with per-tensor scales as TFLOP/s;
  other_configs one duration / throughput / roofline fraction for each remaining benchmark configuration;
  parity        max relative error of one ring entry against the oracle.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_FP8_PEAK_TFLOPS = 5000.0
# HBM bytes one GEMV launch moves come from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` over the --pmc-calibration
# run of this file, each scaled by what the same counter reads for a 64 MiB device copy. The figure is a record of that
# profile, not measured in this run: the summary keeps it in a small JSON block, which is read here and reported together
# with the summary's name.
GEMV_TRAFFIC_PROFILE = 'profiles/skinny_w8a16_gemv_m1_k4096_n11008_hbm_traffic.md'


def measured_gemv_traffic():
    """(bytes per launch or None, the record) from the ```json block of the traffic summary."""
    import re
    try:
        text = open(os.path.join(ROOT, GEMV_TRAFFIC_PROFILE)).read()
        rec = json.loads(re.search(r'```json\s*(\{.*?\})\s*```', text, flags=re.S).group(1))
        return float(rec['hbm_bytes_per_launch']), rec
    except (OSError, AttributeError, KeyError, ValueError):
        return None, None


K, N = 4096, 11008
RING = 16
GEMV_BYTES = K * N + 2 * N + 2 * K + 2 * N  # weights + scales + activations + output, each once


def make_ring(quant, make_inputs, ring, k, n, device):
    """Ring entry i holds the weights of the parity tests' seeded recipe (oracle.make_inputs(seed=i): A ~ N(0, 1) drawn
    first, then W ~ N(0, 0.02^2)), quantized on the GPU by the library (bit-exact with the oracle's quantizer, which the
    GPU tests check at this shape). Seeds 0-3 are the benchmark configuration's; the rest fill the ring."""
    ws, ss, a0 = [], [], None
    for i in range(ring):
        a32, w32 = make_inputs(i, 1, k, n)
        if i == 0:
            a0 = torch.from_numpy(a32).to(device).to(torch.float16)
        wq, s32 = quant.symmetric_quantize(torch.from_numpy(w32).to(device), 'int8', dims=0)
        ws.append(wq)
        ss.append(s32.to(torch.float16))
        del w32
    return a0, ws, ss


def cpu_baseline(a_np, wq_np, s_np, budget_s=12.0):
    from oracle import clib

    threads = clib.lib().oracle_baseline_threads()
    t0 = time.perf_counter()
    clib.baseline_quant_matmul(a_np, wq_np, s_np)
    one = time.perf_counter() - t0
    reps = max(1, min(200, int(budget_s / max(one, 1e-3))))
    t0 = time.perf_counter()
    for _ in range(reps):
        out = clib.baseline_quant_matmul(a_np, wq_np, s_np)
    dt = (time.perf_counter() - t0) / reps
    res = {
        'value': GEMV_BYTES / dt / 1e9, 'unit': 'GB/s', 'cores': int(threads), 'kind': 'port',
        'sample': 'full M=1 K=4096 N=11008 GEMV, {} repetitions, {:.1f} ms each; nproc={}'.format(reps, dt * 1e3, os.cpu_count()),
    }
    # the reference's own CPU-runnable configuration, timed in full: M = 16, K = N = 4096 (same loop nest, same flags)
    rng = np.random.default_rng(0)
    a16 = rng.standard_normal((16, 4096), dtype=np.float32).astype(np.float16)
    w16, s16 = wq_np[:, :4096], s_np[:4096]
    t0 = time.perf_counter()
    clib.baseline_quant_matmul(a16, w16, s16)
    c1 = time.perf_counter() - t0
    c1_bytes = 4096 * 4096 + 2 * 4096 + 2 * 2 * 16 * 4096
    res['m16_k4096_n4096_full'] = {'seconds': round(c1, 4), 'GB/s': round(c1_bytes / c1 / 1e9, 3), 'GFLOP/s': round(2 * 16 * 4096 * 4096 / c1 / 1e9, 2)}
    # best effort on the same cores: dequantize once, then torch.matmul in fp32 (what a CPU user would really run); the
    # headline GEMV shape, weights already dequantized outside the timed region
    torch.set_num_threads(int(threads))
    wt = torch.from_numpy(wq_np).float() * torch.from_numpy(s_np.astype(np.float32))
    at = torch.from_numpy(a_np.astype(np.float32))
    torch.matmul(at, wt)
    t0 = time.perf_counter()
    for _ in range(20):
        torch.matmul(at, wt)
    tm = (time.perf_counter() - t0) / 20
    res['best_effort_torch_matmul_fp32'] = {'seconds': round(tm, 5), 'GB/s_of_int8_bytes': round(GEMV_BYTES / tm / 1e9, 2),
                                            'threads': int(threads), 'note': 'fp32 weights dequantized beforehand; 4 x the bytes of the int8 path'}
    return res, out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--pmc-calibration', action='store_true',
                    help='short run for `rocprofv3 --pmc`: a few 64 MiB device copies of known traffic, then one pass over the GEMV ring')
    ap.add_argument('--decode-counters', action='store_true',
                    help='short run for `rocprofv3 --pmc`: the decode kernels of the smaller configurations only (W4A16 M = 1 and 16 '
                         'at 4096 x 11008, W8A16 M = 16 at 4096 x 4096, the headline GEMV for comparison), over distinct weight buffers')
    ap.add_argument('--skip-two-chains', action='store_true',
                    help='leave out the two-stream graph: under a kernel trace its overlapping launches would blur the GEMV kernel\'s average duration')
    ap.add_argument('--skip-exchange-probe', action='store_true',
                    help='leave out the GEMV passes with a poll limit of zero (launches that never wait for the exchange): under a '
                         'kernel trace they cannot be told from the measured launches and would pull the kernel\'s average down')
    ap.add_argument('--data-dependence', action='store_true',
                    help='time the two GEMM kernels on all-zero operands and on the benchmark operands: the instruction '
                         'stream is identical, the difference is the clock the chip sustains under its power limit')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: the quantized-matmul path is built and measured on a single MI355X '
              '(--gpus {} is not supported)'.format(args.gpus), file=sys.stderr)
        sys.exit(2)

    import hidet_amd
    from hidet_amd import ffi
    from hidet_amd.graph.ops import quant

    device = torch.device('cuda:0')
    torch.cuda.set_device(device)
    lib = ffi.load_library()

    from oracle import oracle as O
    g = torch.Generator(device=device)
    g.manual_seed(1234)
    a, ws, ss = make_ring(quant, O.make_inputs, RING, K, N, device)
    outs = [torch.empty((1, N), dtype=torch.float16, device=device) for _ in range(RING)]
    work = ffi.workspace(device)

    stream = torch.cuda.Stream(device)
    sptr = stream.cuda_stream

    def launch(i, st):
        ffi.call('hidet_symmetric_quant_matmul_f16_i8', a, ws[i], ss[i], outs[i], 1, K, N, K, 0, work, work.numel(), st)

    if args.decode_counters:
        g2 = torch.Generator(device=device)
        g2.manual_seed(7)
        w4 = [torch.randint(0, 256, (K, N // 2), device=device, dtype=torch.uint8) for _ in range(16)]
        s4 = (torch.rand((K // 128, N), generator=g2, device=device) * 0.01 + 0.001).to(torch.bfloat16)
        w16 = [torch.randint(-127, 128, (4096, 4096), device=device, dtype=torch.int8) for _ in range(16)]
        a16 = torch.randn((16, 4096), generator=g2, device=device, dtype=torch.float32).to(torch.float16)
        c16 = torch.empty((16, 4096), dtype=torch.float16, device=device)
        s16 = ss[0][:4096].contiguous()
        with torch.cuda.stream(stream):
            for m4 in (1, 16):
                a4 = torch.randn((m4, K), generator=g2, device=device, dtype=torch.float32).to(torch.bfloat16)
                c4 = torch.empty((m4, N), dtype=torch.bfloat16, device=device)
                for rep in range(2):
                    for i in range(16):
                        ffi.call('hidet_symmetric_quant_matmul_w4a16', a4, w4[i], s4, c4, m4, K, N, K, 128, 2, 0, work, work.numel(), sptr)
            for rep in range(2):
                for i in range(16):
                    ffi.call('hidet_symmetric_quant_matmul_f16_i8', a16, w16[i], s16, c16, 16, 4096, 4096, 4096, 0, work, work.numel(), sptr)
            for rep in range(2):
                for i in range(RING):
                    launch(i, sptr)
        stream.synchronize()
        print(json.dumps({'decode_counters': {'order': ['w4a16 m=1 x32', 'w4a16 m=16 x32', 'w8a16 m=16 4096x4096 x32', 'w8a16 gemv x32']}}))
        return

    if args.pmc_calibration:
        src = torch.empty(64 << 20, dtype=torch.uint8, device=device).random_(0, 255)
        dst = torch.empty_like(src)
        with torch.cuda.stream(stream):
            for _ in range(4):
                dst.copy_(src)  # 64 MiB read + 64 MiB written per dispatch
            for rep in range(2):
                for i in range(RING):
                    launch(i, sptr)
            # the same ring read as K-contiguous [N, K] weights by the kernel for that layout (other_configs)
            c_nk = torch.empty((1, N), dtype=torch.float16, device=device)
            for rep in range(2):
                for i in range(RING):
                    ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', a, ws[i].view(N, K), ss[0], c_nk, 1, K, N, K, K, None, 0, sptr)
        stream.synchronize()
        print(json.dumps({'pmc_calibration': {'copy_bytes': 64 << 20, 'copies': 4, 'gemv_launches': 2 * RING,
                                              'gemv_k_contiguous_launches': 2 * RING, 'gemv_algorithmic_bytes': GEMV_BYTES}}))
        return

    # ---- parity of one ring entry against the oracle, before anything is timed --------------------------
    from oracle import clib
    with torch.cuda.stream(stream):
        launch(3, sptr)
    stream.synchronize()
    a_np, w_np, s_np = a.cpu().numpy(), ws[3].cpu().numpy(), ss[3].cpu().numpy()
    ref = clib.quant_matmul_f32acc(a_np, w_np, s_np)
    parity = O.max_rel_err(outs[3].cpu().numpy(), ref)

    # ---- one step = one pass over the ring, captured as a HIP graph ---------------------------------------
    with torch.cuda.stream(stream):
        for i in range(RING):
            launch(i, sptr)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        cs = torch.cuda.current_stream(device).cuda_stream
        for i in range(RING):
            launch(i, cs)
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.replay()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = RING * GEMV_BYTES / (ms_per_step * 1e-3) / 1e9

    # replayed results still match the eager ones
    replay_ok = bool(O.max_rel_err(outs[3].cpu().numpy(), ref) == parity)

    # ---- the same 16 launches as two independent chains of 8 on two streams of one graph (each with its own workspace):
    # what two projections that do not depend on each other (gate and up of one MLP, or q / k / v) get when they overlap.
    # Reported next to `value`, which stays the single dependent chain.
    two_chains = None
    side = [] if args.skip_two_chains else [torch.cuda.Stream(device), torch.cuda.Stream(device)]
    if side:
        side_work = []
        for st in side:
            with torch.cuda.stream(st):
                side_work.append(ffi.workspace(device))
        torch.cuda.synchronize()

        def launch_pairs():
            for i in range(RING):
                wk = side_work[i & 1]
                ffi.call('hidet_symmetric_quant_matmul_f16_i8', a, ws[i], ss[i], outs[i], 1, K, N, K, 0, wk, wk.numel(),
                         side[i & 1].cuda_stream)

        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2, stream=stream):
            for st in side:
                st.wait_stream(stream)
            launch_pairs()
            for st in side:
                stream.wait_stream(st)
        for _ in range(args.warmup):
            graph2.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph2.replay()
        torch.cuda.synchronize()
        pair_ms = (time.perf_counter() - t0) / args.steps * 1e3
        pair_ok = bool(O.max_rel_err(outs[3].cpu().numpy(), ref) == parity)
        two_chains = {'workload': 'the same 16 GEMVs as two independent chains of 8 on two streams of one graph',
                      'ms_per_step': round(pair_ms, 5), 'GB/s': round(RING * GEMV_BYTES / (pair_ms * 1e-3) / 1e9, 1),
                      'frac_of_hbm_peak': round(RING * GEMV_BYTES / (pair_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                      'matches_eager': pair_ok}

    # ---- the kernel's own duration: begin/end of every dispatch through the timing hook, the ring launched back to
    # back as in the timed region (each launch has its own pair of events; one synchronisation per pass) -------------
    LAPS = 4  # the ring this many times per pass, back to back: 64 consecutive launches between two synchronisations
    import ctypes
    evs = [(lib.hidet_qmm_event_create(), lib.hidet_qmm_event_create()) for _ in range(LAPS * RING)]
    ptr_array = ctypes.c_void_p * RING
    ev_array = ctypes.c_void_p * (LAPS * RING)
    w_ptrs, s_ptrs, o_ptrs = (ptr_array(*[t.data_ptr() for t in ts]) for ts in (ws, ss, outs))
    e0s, e1s = ev_array(*[e[0] for e in evs]), ev_array(*[e[1] for e in evs])
    def native_passes(passes):
        durs = []
        for rep in range(passes):
            # one native loop per pass: an untimed lap (the pass starts behind a synchronisation, the timed region does not),
            # then the timed launches. Issued from Python one call at a time, a launch costs the host about as long as the
            # kernel runs, and on a slow host the stream's queue runs dry in the later laps of a pass: the kernels then start
            # on an idle memory system and take 0.5-1.5 us longer (seen as a mean that grows from lap to lap)
            ffi.call('hidet_qmm_gemv_ring_timed', a, w_ptrs, s_ptrs, o_ptrs, RING, RING, 1, K, N, K, work, work.numel(), None, None, sptr)
            ffi.call('hidet_qmm_gemv_ring_timed', a, w_ptrs, s_ptrs, o_ptrs, RING, LAPS * RING, 1, K, N, K, work, work.numel(), e0s, e1s, sptr)
            stream.synchronize()
            durs.extend(lib.hidet_qmm_event_elapsed_ms(e0, e1) * 1e3 for e0, e1 in evs)
        return np.array(durs[LAPS * RING:])  # first pass warms the instruction cache

    durs = native_passes(5)
    kernel_us = float(durs.mean())
    # What waiting for the exchange costs: the same passes with the collectors' poll limit at zero - they read the mailbox
    # once and give up (outputs NaN, a flag in the workspace), so no launch waits for a partial tile. Afterwards the limit
    # goes back to its default, the workspace is put back in order, and a launch must give the parity result again.
    no_wait_us = None
    if not args.skip_exchange_probe:
        lib.hidet_qmm_set_exchange_spin_limit(0)
        no_wait_us = float(native_passes(3).mean())
        lib.hidet_qmm_set_exchange_spin_limit(-1)
        gave_up = lib.hidet_qmm_exchange_status(work.data_ptr(), work.numel(), sptr)
        lib.hidet_qmm_exchange_reset(work.data_ptr(), work.numel(), sptr)
        launch(3, sptr)
        stream.synchronize()
        if gave_up != 1 or O.max_rel_err(outs[3].cpu().numpy(), ref) != parity:
            raise SystemExit('bench.py: the exchange did not recover after the run without waiting')
    for e0, e1 in evs:
        lib.hidet_qmm_event_destroy(e0)
        lib.hidet_qmm_event_destroy(e1)
    # where the slow launches are: by weight buffer (physical placement of a 45 MB buffer), by position in a pass
    # (a pass starts behind one untimed lap), by pass
    by_launch = durs.reshape(-1, LAPS, RING)
    slow = durs > 1.2 * np.median(durs)
    spread = {'p90': round(float(np.percentile(durs, 90)), 3), 'p99': round(float(np.percentile(durs, 99)), 3),
              'max': round(float(durs.max()), 3),
              'mean_by_weight_buffer': [round(float(x), 2) for x in by_launch.mean(axis=(0, 1))],
              'mean_by_lap_of_a_pass': [round(float(x), 2) for x in by_launch.mean(axis=(0, 2))],
              'mean_by_pass': [round(float(x), 2) for x in by_launch.mean(axis=(1, 2))],
              'launches_over_1.2_x_p50': int(slow.sum()),
              'of_them_by_weight_buffer': [int(x) for x in slow.reshape(-1, LAPS, RING).sum(axis=(0, 1))]}
    achieved = GEMV_BYTES / (kernel_us * 1e-6) / 1e9

    # single-buffer (last-level-cache-hot) figure, labelled as such
    with torch.cuda.stream(stream):
        for _ in range(50):
            launch(0, sptr)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(500):
            launch(0, sptr)
        e1.record(stream)
    e1.synchronize()
    hot_us = e0.elapsed_time(e1) / 500 * 1e3

    def time_gemm_series(launch_one, reps=24, skip=4):
        """Kernel durations (us) of a GEMM, two ways, each started on a chip that has idled for a second (what ran before
        in this process must not decide the clock a series gets). The figure reported: one launch at a time, each waited
        for before the next goes out, as in the earlier records of this benchmark. Next to it the same number of launches
        back to back, each with its own pair of events: the rate under sustained load. Which of the two is faster depends
        on the box (the chip runs these kernels at its power limit, and the gaps of the first form let it recover)."""
        def rest():
            torch.cuda.synchronize()
            time.sleep(1.0)
        rest()
        pairs = [(lib.hidet_qmm_event_create(), lib.hidet_qmm_event_create()) for _ in range(reps)]
        for rep, (x0, x1) in enumerate(pairs):
            lib.hidet_qmm_arm_timing(x0, x1)
            launch_one(rep % 3)
        stream.synchronize()
        sustained = [lib.hidet_qmm_event_elapsed_ms(x0, x1) * 1e3 for x0, x1 in pairs]
        for x0, x1 in pairs:
            lib.hidet_qmm_event_destroy(x0)
            lib.hidet_qmm_event_destroy(x1)
        rest()
        e0, e1 = lib.hidet_qmm_event_create(), lib.hidet_qmm_event_create()
        one = []
        for rep in range(reps):
            lib.hidet_qmm_arm_timing(e0, e1)
            launch_one(rep % 3)
            lib.hidet_qmm_event_synchronize(e1)
            one.append(lib.hidet_qmm_event_elapsed_ms(e0, e1) * 1e3)
        lib.hidet_qmm_event_destroy(e0)
        lib.hidet_qmm_event_destroy(e1)
        return np.array(one[skip:]), np.array(sustained[skip:])

    # ---- second half of the metric: the M = 2048 prefill GEMM of the same weight shape ------------------------
    MP = 2048
    gp = torch.Generator(device=device)
    gp.manual_seed(4321)
    ap = torch.randn((MP, K), generator=gp, device=device, dtype=torch.float32).to(torch.float16)
    cp = torch.empty((MP, N), dtype=torch.float16, device=device)

    def launch_prefill(i):
        ffi.call('hidet_symmetric_quant_matmul_f16_i8', ap, ws[i], ss[i], cp, MP, K, N, K, 0, work, work.numel(), sptr)

    with torch.cuda.stream(stream):
        for i in range(3):
            launch_prefill(i)
    stream.synchronize()
    rows = np.array([0, 127, 128, 1029, 2047])
    pref = clib.quant_matmul_f32acc(ap.cpu().numpy()[rows], ws[2].cpu().numpy(), ss[2].cpu().numpy())
    prefill_parity = O.max_rel_err(cp.cpu().numpy()[rows], pref)
    pd, pd_sustained = time_gemm_series(launch_prefill)
    prefill_flops = 2.0 * MP * K * N
    prefill_tflops = prefill_flops / (pd.mean() * 1e-6) / 1e12

    # ---- FP8 e4m3 GEMM with per-tensor scales: a [4096, 8192] ~ N(0, 1), b [8192, 8192] ~ N(0, 0.02), bf16 output ----
    from hidet_amd.graph.ops.matmul import matmul_f8 as f8ops
    MF, KF, NF = 4096, 8192, 8192
    gf = torch.Generator(device=device)
    gf.manual_seed(0)
    a8, sa = f8ops.fp8_quantize_per_tensor(torch.randn((MF, KF), generator=gf, device=device, dtype=torch.float32))
    b8s = []
    for i in range(3):
        bq, sb = f8ops.fp8_quantize_per_tensor(torch.randn((NF, KF), generator=gf, device=device, dtype=torch.float32) * 0.02)
        b8s.append((bq, sb))
    c8 = torch.empty((MF, NF), dtype=torch.bfloat16, device=device)

    def launch_fp8(i):
        ffi.call('hidet_matmul_f8', a8, b8s[i][0], c8, MF, NF, KF, KF, KF, 2, sa, b8s[i][1], work, work.numel(), sptr)

    with torch.cuda.stream(stream):
        for i in range(3):
            launch_fp8(i)
    stream.synchronize()
    rows8 = np.array([0, 255, 256, 2049, 4095])
    ref8 = O.fp8_matmul_per_tensor(a8.view(torch.uint8).cpu().numpy()[rows8], b8s[2][0].view(torch.uint8).cpu().numpy(),
                                   float(sa.cpu()), float(b8s[2][1].cpu()), 'float32')
    fp8_parity = O.max_rel_err(c8.float().cpu().numpy()[rows8], ref8)
    fd, fd_sustained = time_gemm_series(launch_fp8)
    fp8_tflops = 2.0 * MF * KF * NF / (fd.mean() * 1e-6) / 1e12

    # ---- the other benchmark configurations, one figure each (kernel duration through the timing hook, distinct weight
    # buffers per launch so that nothing is served from the last-level cache) ------------------------------------------
    # A spin kernel of about 300 us that a batch of short launches is queued behind: the host needs about as long per call
    # as a decode kernel runs, so without it the stream's queue can run dry inside a batch and the kernels start on an
    # idle memory system. torch's sleep kernel counts a clock whose rate is measured here once.
    with torch.cuda.stream(stream):
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda._sleep(1000)
        t0.record(stream)
        torch.cuda._sleep(1000000)
        t1.record(stream)
    t1.synchronize()
    blocker_cycles = int(300.0 / max(t0.elapsed_time(t1) * 1e3, 1.0) * 1000000)

    def queue_blocker():
        with torch.cuda.stream(stream):
            torch.cuda._sleep(blocker_cycles)

    def time_kernel(fn, reps, skip, short=True):
        # launches go out back to back in batches of 16, each with its own pair of events: the duration of a dispatch
        # in a busy stream, as in a decode step, not that of a kernel started on an idle chip
        pairs = [(lib.hidet_qmm_event_create(), lib.hidet_qmm_event_create()) for _ in range(16)]
        d = []
        for r0 in range(0, reps, 16):
            nb = min(16, reps - r0)
            if short:  # decode-sized kernels; the GEMMs run far longer than the host needs per call
                queue_blocker()
            for j in range(2):  # untimed: a batch starts behind a synchronisation, a decode step does not
                fn(r0 + nb - 1 - j)
            for j in range(nb):
                lib.hidet_qmm_arm_timing(pairs[j][0], pairs[j][1])
                fn(r0 + j)
            stream.synchronize()
            d.extend(lib.hidet_qmm_event_elapsed_ms(pairs[j][0], pairs[j][1]) * 1e3 for j in range(nb))
        for e0, e1 in pairs:
            lib.hidet_qmm_event_destroy(e0)
            lib.hidet_qmm_event_destroy(e1)
        return float(np.mean(d[skip:]))

    def hbm_entry(us, nbytes):
        return {'kernel_us': round(us, 2), 'GB/s': round(nbytes / us / 1e3, 1), 'frac_of_hbm_peak': round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    def mfma_entry(us, flops, peak):
        return {'kernel_us': round(us, 2), 'TFLOP/s': round(flops / us / 1e6, 1), 'frac_of_mfma_peak': round(flops / us / 1e6 / peak, 4)}

    others = {}
    # W8A16, M = 16, 4096 x 4096 (the reference's CPU-runnable case)
    w16 = [torch.randint(-127, 128, (4096, 4096), device=device, dtype=torch.int8) for _ in range(32)]  # 2 x the 256 MB LLC
    s16 = ss[0][:4096].contiguous()
    a16 = torch.randn((16, 4096), generator=g, device=device, dtype=torch.float32).to(torch.float16)
    c16 = torch.empty((16, 4096), dtype=torch.float16, device=device)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', a16, w16[r % 32], s16, c16, 16, 4096, 4096, 4096, 0,
                                      work, work.numel(), sptr), 96, 32)
    others['w8a16_m16_k4096_n4096'] = hbm_entry(us, 4096 * 4096 + 2 * 4096 + 2 * 16 * 4096 * 2)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', a16, w16[r % 32], s16, c16, 16, 4096, 4096, 4096, 4096,
                                      None, 0, sptr), 96, 32)  # the same buffers read as [N, K] storage
    others['w8a16_m16_k4096_n4096_k_contiguous_weights'] = hbm_entry(us, 4096 * 4096 + 2 * 4096 + 2 * 16 * 4096 * 2)
    del w16
    # W8A16 decode GEMV, down-proj shape [1, 11008] x [11008, 4096]: the ring's buffers reinterpreted as [11008, 4096]
    ad = torch.randn((1, N), generator=g, device=device, dtype=torch.float32).to(torch.float16)
    cd = torch.empty((1, K), dtype=torch.float16, device=device)
    sd = ss[0][:K].contiguous()
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', ad, ws[r % RING].view(N, K), sd, cd, 1, N, K, N, 0,
                                      work, work.numel(), sptr), 48, 16)
    others['w8a16_gemv_down_proj_k11008_n4096'] = hbm_entry(us, K * N + 2 * K + 2 * N + 2 * K)
    # the same two GEMVs on weights stored K-contiguous (the [N, K] storage of torch.nn.Linear, passed as a [K, N] view):
    # another data layout than the benchmark configuration's, so never the headline; the ring's buffers reinterpreted
    cu = torch.empty((1, N), dtype=torch.float16, device=device)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', a, ws[r % RING].view(N, K), ss[0], cu, 1, K, N, K, K,
                                      None, 0, sptr), 48, 16)
    others['w8a16_gemv_k4096_n11008_k_contiguous_weights'] = hbm_entry(us, K * N + 2 * K + 2 * N + 2 * N)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', ad, ws[r % RING].view(K, N), sd, cd, 1, N, K, N, N,
                                      None, 0, sptr), 48, 16)
    others['w8a16_gemv_down_proj_k11008_n4096_k_contiguous_weights'] = hbm_entry(us, K * N + 2 * K + 2 * N + 2 * K)
    # the same GEMV on the first 256 ... 2048 rows of the ring's matrices (and all 4096): time against K at N = 11008 separates
    # what a launch costs whatever it reads from what its bytes cost
    sweep = {}
    for kk in (256, 1024, 2048, 4096):
        ak = a[:, :kk].contiguous()
        us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', ak, ws[r % RING], ss[0], cu, 1, kk, N, kk, 0,
                                          work, work.numel(), sptr), 48, 16)
        sweep['k{}'.format(kk)] = round(us, 2)
    others['w8a16_gemv_n11008_us_against_k'] = sweep
    # the same GEMV kernel on a matrix five times the size (not a benchmark configuration: it shows how much of the headline
    # figure is the fixed cost of one launch and one cross-workgroup exchange)
    wl = [torch.randint(-127, 128, (8192, 28672), device=device, dtype=torch.int8) for _ in range(3)]  # 3 x 235 MB > LLC
    al = torch.randn((1, 8192), generator=g, device=device, dtype=torch.float32).to(torch.float16)
    sl = torch.cat([ss[0], ss[1], ss[2]])[:28672].contiguous()
    cl = torch.empty((1, 28672), dtype=torch.float16, device=device)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', al, wl[r % 3], sl, cl, 1, 8192, 28672, 8192, 0,
                                      work, work.numel(), sptr), 24, 6)
    others['w8a16_gemv_k8192_n28672_not_a_baseline_config'] = hbm_entry(us, 8192 * 28672 + 2 * 28672 + 2 * 8192 + 2 * 28672)
    # what a kernel that only reads gets out of the memory system at these two sizes (16-byte loads, 32 KiB contiguous per
    # workgroup, nothing else): the practical ceiling of the decode kernels, next to the data sheet's 8 TB/s
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    us = time_kernel(lambda r: ffi.call('hidet_qmm_read_probe', wl[r % 3], 8192 * 28672, sink, sptr), 24, 6)
    read_probe = {'read_only_kernel_235MB': hbm_entry(us, 8192 * 28672)}
    del wl
    us = time_kernel(lambda r: ffi.call('hidet_qmm_read_probe', ws[r % RING], K * N, sink, sptr), 64, 16)
    read_probe['read_only_kernel_45MB'] = hbm_entry(us, K * N)
    # the loads of the GEMV kernel over the same matrices without its arithmetic and its exchange (256-column tiles, rows
    # in steps of 32, one step per wave in flight), on the 256 workgroups of its launch and on the 172 of a plan of four
    # slices per tile; and the same bytes per wave read as contiguous 1 KiB pieces
    for label, groups, contiguous in (('gemv_access_pattern_256_workgroups', 256, 0), ('gemv_access_pattern_172_workgroups', 172, 0),
                                      ('same_bytes_per_wave_contiguous_256_workgroups', 256, 1)):
        us = time_kernel(lambda r: ffi.call('hidet_qmm_pattern_probe', ws[r % RING], K, N, groups, contiguous, sink, sptr), 64, 16)
        read_probe[label + '_45MB'] = hbm_entry(us, K * N)
    # the GEMV's grid (256 workgroups of 512 threads) with 8 KiB to read in all: what lies between a launch's begin and end
    # events before the matrix moves
    us = time_kernel(lambda r: ffi.call('hidet_qmm_pattern_probe', ws[r % RING], 32, 256, 256, 0, sink, sptr), 64, 16)
    read_probe['launch_of_the_gemv_grid_reading_8_KiB_us'] = round(us, 2)
    read_probe['gemv_with_a_poll_limit_of_zero_us'] = None if no_wait_us is None else round(no_wait_us, 3)
    # W8A16 prefill, attention QKV shape [2048, 4096] x [4096, 12288]
    wq = [torch.randint(-127, 128, (K, 12288), device=device, dtype=torch.int8) for _ in range(4)]
    sq = torch.cat([ss[0], ss[1]])[:12288].contiguous()
    cq = torch.empty((MP, 12288), dtype=torch.float16, device=device)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', ap, wq[r % 4], sq, cq, MP, K, 12288, K, 0, work,
                                      work.numel(), sptr), 16, 4, short=False)
    others['w8a16_prefill_m2048_k4096_n12288'] = mfma_entry(us, 2.0 * MP * K * 12288, MFMA_F16_PEAK_TFLOPS)
    # the M = 2048 prefill GEMM on K-contiguous weights (the ring's buffers read as [N, K] storage; another layout), and 32 rows
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', ap, ws[r % RING].view(N, K), ss[0], cp, MP, K, N, K, K,
                                      work, work.numel(), sptr), 16, 4, short=False)
    others['w8a16_prefill_m2048_k4096_n11008_k_contiguous_weights'] = mfma_entry(us, 2.0 * MP * K * N, MFMA_F16_PEAK_TFLOPS)
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', ap[:32], ws[r % RING].view(N, K), ss[0], cp[:32], 32, K, N,
                                      K, K, work, work.numel(), sptr), 32, 16)
    others['w8a16_m32_k4096_n11008_k_contiguous_weights'] = hbm_entry(us, K * N + 2 * N + 2 * 32 * (K + N))
    us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', ap[:32], ws[r % RING], ss[0], cp[:32], 32, K, N, K, 0,
                                      work, work.numel(), sptr), 32, 16)
    others['w8a16_m32_k4096_n11008'] = hbm_entry(us, K * N + 2 * N + 2 * 32 * (K + N))
    del wq, cq
    # group-wise W4A16 (bf16, group 128), M in {1, 16, 512}
    w4 = [torch.randint(0, 256, (K, N // 2), device=device, dtype=torch.uint8) for _ in range(24)]  # 24 x 22.5 MB = 541 MB > 2 x the LLC
    s4 = (torch.rand((K // 128, N), generator=g, device=device) * 0.01 + 0.001).to(torch.bfloat16)
    for m4 in (1, 16, 512):
        a4 = torch.randn((m4, K), generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
        c4 = torch.empty((m4, N), dtype=torch.bfloat16, device=device)
        us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_w4a16', a4, w4[r % 24], s4, c4, m4, K, N, K, 128, 2, 0,
                                          work, work.numel(), sptr), 48, 24, short=m4 <= 16)
        nbytes = K * N // 2 + 2 * (K // 128) * N + 2 * m4 * K + 2 * m4 * N
        others['w4a16_m{}_k4096_n11008'.format(m4)] = (hbm_entry(us, nbytes) if m4 <= 16 else
                                                      mfma_entry(us, 2.0 * m4 * K * N, MFMA_F16_PEAK_TFLOPS))
        if m4 <= 16:  # the same bytes read as the [N, K/2] decode layout (another data layout: never the headline)
            us = time_kernel(lambda r: ffi.call('hidet_symmetric_quant_matmul_w4a16_nk', a4, w4[r % 24].view(N, K // 2), s4, c4, m4, K, N,
                                              K, K // 2, 128, 2, sptr), 48, 24)
            others['w4a16_m{}_k4096_n11008_decode_layout'.format(m4)] = hbm_entry(us, nbytes)
    del w4
    # FP8 decode variant: M = 1 against the same b
    a1 = a8[:1].contiguous()
    c1 = torch.empty((1, NF), dtype=torch.bfloat16, device=device)
    bring = [bq for bq, _ in b8s] + [torch.randint(0, 0x7F, (NF, KF), device=device, dtype=torch.uint8) for _ in range(5)]  # 8 x 64 MiB
    us = time_kernel(lambda r: ffi.call('hidet_matmul_f8', a1, bring[r % 8], c1, 1, NF, KF, KF, KF, 2, sa, b8s[0][1], work, work.numel(), sptr), 32, 8)
    others['fp8_gemv_m1_k8192_n8192'] = hbm_entry(us, NF * KF + KF + 2 * NF + 8)
    # the block-scaled form of the same GEMV (scale_a f32 [K/128, 1], scale_b f32 [N/128, K/128])
    bsa = torch.rand((KF // 128, 1), generator=g, device=device, dtype=torch.float32) + 0.5
    bsb = torch.rand((NF // 128, KF // 128), generator=g, device=device, dtype=torch.float32) + 0.5
    us = time_kernel(lambda r: ffi.call('hidet_matmul_f8_scaled', a1, bring[r % 8], bsa, bsb, c1, 1, NF, KF, 2, work, work.numel(),
                                      sptr), 32, 8)
    others['fp8_block_scaled_gemv_m1_k8192_n8192'] = hbm_entry(us, NF * KF + KF + 2 * NF + 4 * (KF // 128) * (1 + NF // 128))
    del bring

    if args.data_dependence:
        az, wz = torch.zeros_like(ap), torch.zeros_like(ws[0])
        a8z, b8z = torch.zeros_like(a8.view(torch.uint8)), torch.zeros_like(b8s[0][0].view(torch.uint8))
        w8_zero = float(time_gemm_series(lambda r: ffi.call('hidet_symmetric_quant_matmul_f16_i8', az, wz, ss[0], cp, MP, K, N, K, 0, work,
                                                            work.numel(), sptr))[0].mean())
        f8_zero = float(time_gemm_series(lambda r: ffi.call('hidet_matmul_f8', a8z, b8z, c8, MF, NF, KF, KF, KF, 2, sa, b8s[0][1], work,
                                                            work.numel(), sptr))[0].mean())
        print(json.dumps({'data_dependence': {
            'w8a16_gemm_us': {'benchmark_operands': round(float(pd.mean()), 2), 'zero_operands': round(w8_zero, 2)},
            'fp8_gemm_us': {'benchmark_operands': round(float(fd.mean()), 2), 'zero_operands': round(f8_zero, 2)}}}))
        return

    traffic_bytes, traffic_record = measured_gemv_traffic()
    result = {
        'metric': 'w8a16_decode_gemv_bandwidth', 'value': round(value, 1), 'unit': 'GB/s', 'n_gpus': 1,
        'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 5), 'higher_is_better': True,
        'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f16 x int8 -> f32 accumulate', 'data': 'synthetic',
        'config': {'workload': 'W8A16 decode GEMV, a f16[1,4096] x w int8[4096,11008] + f16 scales[11008] -> f16[1,11008]',
                   'inputs': 'oracle.make_inputs(seed) for seeds 0-15 (0-3: the benchmark configuration), weights quantized on the GPU',
                   'launches_per_step': RING, 'distinct_weight_buffers': RING, 'bytes_per_launch': GEMV_BYTES,
                   'graph_replay': True},
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBS, 4), 'traffic': traffic_bytes,
                     'traffic_source': GEMV_TRAFFIC_PROFILE, 'traffic_record': traffic_record, 'algorithmic_bytes': GEMV_BYTES,
                     'duration_of': 'every launch of four laps of the ring, launched back to back from one native loop behind one untimed lap, begin/end of its own dispatch',
                     'kernel': 'skinny_w8a16_kernel', 'kernel_us_mean': round(kernel_us, 3),
                     'kernel_us_min': round(float(durs.min()), 3), 'kernel_us_p50': round(float(np.median(durs)), 3),
                     'launches_timed': int(durs.size), 'spread_us': spread},
        'llc_hot_single_buffer': {'us_per_launch_back_to_back': round(hot_us, 3),
                                  'GB/s': round(GEMV_BYTES / (hot_us * 1e-6) / 1e9, 1)},
        'prefill': {'workload': 'W8A16 prefill GEMM, a f16[2048,4096] x w int8[4096,11008] -> f16[2048,11008]',
                    'value': round(prefill_tflops, 1), 'unit': 'TFLOP/s', 'kernel': 'gemm_w8a16_kernel',
                    'kernel_us_mean': round(float(pd.mean()), 2), 'kernel_us_p50': round(float(np.median(pd)), 2),
                    'kernel_us_min': round(float(pd.min()), 2),
                    'timing': 'one launch at a time after a second of idle, begin/end of each dispatch',
                    'back_to_back_20_launches': {'kernel_us_mean': round(float(pd_sustained.mean()), 2),
                                                 'TFLOP/s': round(prefill_flops / (pd_sustained.mean() * 1e-6) / 1e12, 1),
                                                 'frac': round(prefill_flops / (pd_sustained.mean() * 1e-6) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)},
                    'roofline': {'bound': 'mfma', 'achieved': round(prefill_tflops, 1), 'peak': MFMA_F16_PEAK_TFLOPS,
                                 'unit': 'TFLOP/s', 'frac': round(prefill_tflops / MFMA_F16_PEAK_TFLOPS, 4)},
                    'max_rel_err_vs_oracle_rows_sample': prefill_parity},
        'fp8_prefill': {'workload': 'FP8 e4m3 GEMM, a[4096,8192] x b[8192,8192]^T, per-tensor f32 scales -> bf16[4096,8192]',
                        'value': round(fp8_tflops, 1), 'unit': 'TFLOP/s', 'kernel': 'gemm_fp8_kernel',
                        'kernel_us_mean': round(float(fd.mean()), 2), 'kernel_us_p50': round(float(np.median(fd)), 2),
                        'kernel_us_min': round(float(fd.min()), 2),
                        'timing': 'one launch at a time after a second of idle, begin/end of each dispatch',
                        'back_to_back_20_launches': {'kernel_us_mean': round(float(fd_sustained.mean()), 2),
                                                     'TFLOP/s': round(2.0 * MF * KF * NF / (fd_sustained.mean() * 1e-6) / 1e12, 1),
                                                     'frac': round(2.0 * MF * KF * NF / (fd_sustained.mean() * 1e-6) / 1e12 / MFMA_FP8_PEAK_TFLOPS, 4)},
                        'roofline': {'bound': 'mfma', 'achieved': round(fp8_tflops, 1), 'peak': MFMA_FP8_PEAK_TFLOPS,
                                     'unit': 'TFLOP/s', 'frac': round(fp8_tflops / MFMA_FP8_PEAK_TFLOPS, 4)},
                        'max_rel_err_vs_oracle_rows_sample': fp8_parity, 'tolerance': 3e-2},
        'two_independent_chains': two_chains,
        'other_configs': others,
        'read_probe': read_probe,
        'parity': {'max_rel_err_vs_oracle': parity, 'tolerance': 1e-2, 'graph_replay_matches_eager': replay_ok},
    }
    if not args.no_cpu_baseline:
        result['cpu_baseline'], base_out = cpu_baseline(a_np, w_np, s_np)
        result['cpu_baseline']['max_rel_err_vs_oracle'] = O.max_rel_err(base_out, ref)
    print(json.dumps(result))


if __name__ == '__main__':
    main()
