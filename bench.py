#!/usr/bin/env python3
"""Benchmark of the RWKV7 generalized delta rule on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch of synthetic input: the chunked
prefill `generalized_delta_rule` call at B=8, T=4096, H=32, K=V=64, bf16 inputs, float32
initial state in, final state out (the RWKV7-1.5B layer shape).  Inputs are resident in
HBM before the timed region.  Prints ONE JSON line:

  metric/value   prefill tokens/s (B*T tokens per step)
  roofline       algorithmic bytes of one step / measured step time against the 8 TB/s HBM
                 peak (the operator is a scan: HBM is its binding roofline), with the step's
                 one kernel also timed alone by events on the launch stream
  mfma           algorithmic and executed bf16 MFMA TFLOP/s against the 2.5 PFLOP/s dense peak
  decode         T=1 decode at B=256, H=40: 64 consecutive in-place steps, state GB/s
  cpu_baseline   the CPU restatement of the reference's native loop, timed on this host

This file only measures; the parity checks live in tests/.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12            # B/s, MI355X HBM3E
MFMA_BF16_PEAK = 2.5e15      # flop/s, dense bf16

PREFILL = dict(B=8, T=4096, H=32)          # chunked prefill, RWKV7-1.5B layer shape
DECODE = dict(B=256, H=40, steps=64)       # T = 1 decode, RWKV7-2.9B shape
PREWARM_STEPS = 150                        # untimed steps that bring the GPU to its steady clocks
BACKWARD = dict(B=4, T=2048, H=32)         # the reference's 4-GPU training shape, one GPU's share
N = 64

# Bytes beyond L2 per step (the one fused chunk_summary_kernel<2> launch) measured with
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` on this same command, each scaled by what the
# counter reads for a plain 1 GiB copy (FETCH_SIZE x2.000, WRITE_SIZE x1.000); the summary is
# profiles/fwd_chunk_prefill_and_decode_traffic.txt.
MEASURED_TRAFFIC_BYTES = 1536130562
TRAFFIC_SOURCE = ("profiles/fwd_chunk_prefill_and_decode_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this "
                  "command at B=8 T=4096 H=32; a constant, not measured in this run)")
EXEC_FLOPS_SOURCE = ("profiles/fwd_chunk_prefill_mfma_counters.txt (SQ_INSTS_VALU_MFMA_MOPS_BF16: 118,784 flop per "
                     "token-head; a constant, not measured in this run)")


# The two constants above describe the kernels as they were when the profiles were taken: the digest of the
# kernel sources (sources_digest() below) at that time.  The JSON line carries this digest next to the digest of
# the sources in the tree and of the loaded library, so a reader sees whether the constants still belong to
# the code that was timed.
CONSTANTS_SOURCES_DIGEST = "55ac6daa92b2ca87"


def sources_digest():
    """sha256 (first 16 hex digits) over the kernel sources and the C-ABI headers, in name order."""
    import glob
    import hashlib
    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(ROOT, "rwkv_ops_amd", "csrc", "*.hip")) +
                   glob.glob(os.path.join(ROOT, "rwkv_ops_amd", "csrc", "*.h")) +
                   glob.glob(os.path.join(ROOT, "include", "*.h")))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def file_digest(path):
    import hashlib
    with open(path, "rb") as fh:
        return hashlib.sha256(fh.read()).hexdigest()[:16]


def algorithmic_bytes_prefill(B, T, H):
    # r, w, k, v, a, b read + o written (bf16), state read + written (float32)
    return 7 * B * T * H * N * 2 + 2 * B * H * N * N * 4


def algorithmic_bytes_decode(B, H):
    return 2 * B * H * N * N * 4 + 7 * B * H * N * 2


def time_gpu(fn, steps, warmup, torch):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return e0.elapsed_time(e1) / steps, wall_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 1 GiB device copy (the calibration kernel for the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this operator library runs on ONE GPU; --gpus must be 1 "
              "(batch and head sharding need no communication and are left to the caller)",
              file=sys.stderr)
        return 2

    import torch
    import rwkv_ops_amd
    from rwkv_ops_amd.rwkv7 import _lib
    from rwkv_ops_amd.synthetic import make_inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    lib = _lib.load()
    props = torch.cuda.get_device_properties(0)

    # ------------------------------------------------------------------ prefill (the step)
    B, T, H = PREFILL["B"], PREFILL["T"], PREFILL["H"]
    xs = make_inputs(B, T, H, N, seed=1235, dtype=torch.bfloat16)
    r, w, k, v, a, b, h0 = [x.to(dev) for x in xs]
    fn = rwkv_ops_amd.generalized_delta_rule

    def step():
        return fn(r, w, k, v, a, b, h0)

    # The GPU takes a few tens of milliseconds of load to reach its steady clocks (the first ~100 steps
    # after an idle start run up to 10 % slower), so the device is brought there first, whatever
    # --warmup says; the W warm-up steps and the K timed steps follow.
    for _ in range(PREWARM_STEPS):
        step()
    torch.cuda.synchronize()
    ms_step, wall_ms = time_gpu(step, args.steps, args.warmup, torch)
    tokens_per_s = B * T / (ms_step * 1e-3)

    # the step's kernels alone (no tensor allocation around them), with events on the stream they are
    # launched on: rwkv7_fwd = one chunk_summary_kernel<MODE_FUSED> launch
    stream = torch.cuda.current_stream().cuda_stream
    ptr = lambda t: t.data_ptr()
    o = torch.empty_like(r)
    ht = torch.empty(B, H, N, N, dtype=torch.float32, device=dev)
    fws_bytes = lib.rwkv7_fwd_workspace_bytes(B, T, H, 0)
    fws = torch.empty(fws_bytes, dtype=torch.uint8, device=dev)

    def fused():
        rc = lib.rwkv7_fwd(ptr(r), ptr(w), ptr(k), ptr(v), ptr(a), ptr(b), ptr(h0), H * N * N, ptr(o), ptr(ht),
                           B, T, H, N, N, 0, ptr(fws), fws_bytes, stream)
        assert rc == 0, rc

    ms_fused, _ = time_gpu(fused, args.steps, 3, torch)

    # the same forward in its two-kernel form (per-chunk summaries in HBM, then the scan)
    ws_bytes = lib.rwkv7_fwd_chunk_workspace_bytes(B, T, H, 0)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def summary():
        rc = lib.rwkv7_fwd_chunk_summary(ptr(r), ptr(w), ptr(k), ptr(v), ptr(a), ptr(b),
                                         B, T, H, N, N, 0, ptr(ws), ws_bytes, stream)
        assert rc == 0, rc

    def scan():
        rc = lib.rwkv7_fwd_chunk_scan(ptr(h0), H * N * N, ptr(o), ptr(ht), B, T, H, N, N, 0,
                                      ptr(ws), ws_bytes, stream)
        assert rc == 0, rc

    ms_summary, _ = time_gpu(summary, args.steps, 3, torch)
    ms_scan, _ = time_gpu(scan, args.steps, 3, torch)
    del ws

    alg_bytes = algorithmic_bytes_prefill(B, T, H)
    achieved = alg_bytes / (ms_step * 1e-3)
    alg_flops = 9 * N * N * B * T * H                       # 9 K V per token-head
    # executed by the chunk-64 design per token-head, from the SQ_INSTS_VALU_MFMA_MOPS_BF16 counter
    # (profiles/fwd_chunk_prefill_mfma_counters.txt) -- reported separately, never mixed into `achieved`
    exec_flops = 118_784 * B * T * H

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------------ decode
    Bd, Hd, nsteps = DECODE["B"], DECODE["H"], DECODE["steps"]
    xd = make_inputs(Bd, nsteps, Hd, N, seed=1236, dtype=torch.bfloat16)
    seqs = [t.to(dev).permute(1, 0, 2, 3).contiguous() for t in xd[:6]]     # [steps][B,H,64]
    state = xd[6].to(dev).clone()
    od = torch.empty(Bd, Hd, N, dtype=torch.bfloat16, device=dev)

    # per-step argument tuples are built once: the loop below must not be bound by host work
    step_ptrs = [tuple(ptr(s[t]) for s in seqs) for t in range(nsteps)]
    p_state, p_od, stride_d = ptr(state), ptr(od), Hd * N * N
    dec = lib.rwkv7_decode_step

    def decode_64():
        for t in range(nsteps):
            rc = dec(*step_ptrs[t], p_state, stride_d, p_od, p_state, Bd, Hd, N, N, 0, stream)
        assert rc == 0, rc

    ms_dec, _ = time_gpu(decode_64, max(5, args.steps // 5), 3, torch)
    us_per_decode_step = ms_dec * 1e3 / nsteps
    dec_bytes = algorithmic_bytes_decode(Bd, Hd)
    dec_rate = dec_bytes / (us_per_decode_step * 1e-6)
    # the same 64 steps rotating over four states (672 MB, more than the 256 MB memory-side cache):
    # what a model with many layers sees, where a layer's state is evicted between its steps
    states = [state] + [state.clone() for _ in range(3)]

    p_states = [ptr(st) for st in states]

    def decode_64_rot():
        for t in range(nsteps):
            p_st = p_states[t & 3]
            rc = dec(*step_ptrs[t], p_st, stride_d, p_od, p_st, Bd, Hd, N, N, 0, stream)
        assert rc == 0, rc

    ms_rot, _ = time_gpu(decode_64_rot, max(5, args.steps // 5), 3, torch)
    us_rot = ms_rot * 1e3 / nsteps
    del states

    # ------------------------------------------------------------------ backward (training shape)
    Bb, Tb, Hb = BACKWARD["B"], BACKWARD["T"], BACKWARD["H"]
    xb = [x.to(dev) for x in make_inputs(Bb, Tb, Hb, N, seed=1237, dtype=torch.bfloat16)]
    gen = torch.Generator(device="cpu").manual_seed(1238)
    d_o = torch.randn(Bb, Tb, Hb, N, generator=gen).to(torch.bfloat16).to(dev)
    d_ht = (0.1 * torch.randn(Bb, Hb, N, N, generator=gen)).to(dev)
    grads = [torch.empty_like(xb[0]) for _ in range(6)]
    dh0 = torch.empty_like(xb[6])
    bws_bytes = lib.rwkv7_bwd_workspace_bytes(Bb, Tb, Hb, 0)
    bws = torch.empty(bws_bytes, dtype=torch.uint8, device=dev)
    ob = torch.empty_like(xb[0])
    htb = torch.empty_like(xb[6])
    fwsb_bytes = lib.rwkv7_fwd_workspace_bytes(Bb, Tb, Hb, 0)
    fwsb = torch.empty(fwsb_bytes, dtype=torch.uint8, device=dev)

    def bwd():
        rc = lib.rwkv7_bwd(*[ptr(t) for t in xb[:6]], ptr(xb[6]), Hb * N * N, ptr(d_o), ptr(d_ht),
                           *[ptr(g) for g in grads], ptr(dh0), Bb, Tb, Hb, N, N, 0, ptr(bws), bws_bytes, stream)
        assert rc == 0, rc

    def fwd_b():
        rc = lib.rwkv7_fwd(*[ptr(t) for t in xb[:6]], ptr(xb[6]), Hb * N * N, ptr(ob), ptr(htb),
                           Bb, Tb, Hb, N, N, 0, ptr(fwsb), fwsb_bytes, stream)
        assert rc == 0, rc

    ms_bwd, _ = time_gpu(bwd, args.steps, 3, torch)
    ms_fwd_b, _ = time_gpu(fwd_b, args.steps, 3, torch)
    # r, w, k, v, a, b, d_o read + six gradients written (bf16); h0, d_ht read + dh0 written (float32)
    bwd_bytes = 13 * Bb * Tb * Hb * N * 2 + 3 * Bb * Hb * N * N * 4
    del bws, fwsb

    # ------------------------------------------------------------------ packed sequences (cu_seqlens)
    # the prefill step's 32,768 tokens as 64 sequences of random lengths in one packed row
    import random
    rnd = random.Random(1239)
    cuts = sorted(rnd.sample(range(1, B * T), 63))
    cu_host = [0] + cuts + [B * T]
    n_seq = len(cu_host) - 1
    cu = torch.tensor(cu_host, dtype=torch.int32, device=dev)
    h0p = h0[:1].expand(n_seq, -1, -1, -1).contiguous()
    htp = torch.empty_like(h0p)
    pws_bytes = lib.rwkv7_fwd_varlen_workspace_bytes(n_seq, B * T, H, 0)
    pws = torch.empty(pws_bytes, dtype=torch.uint8, device=dev)

    def packed_fwd():
        rc = lib.rwkv7_fwd_varlen(ptr(r), ptr(w), ptr(k), ptr(v), ptr(a), ptr(b), ptr(cu), n_seq, ptr(h0p),
                                  H * N * N, ptr(o), ptr(htp), B * T, H, N, N, 0, ptr(pws), pws_bytes, stream)
        assert rc == 0, rc

    ms_packed_fwd, _ = time_gpu(packed_fwd, args.steps, 3, torch)
    del pws
    pbws_bytes = lib.rwkv7_bwd_varlen_workspace_bytes(n_seq, B * T, H, 0)
    pbws = torch.empty(pbws_bytes, dtype=torch.uint8, device=dev)
    pgrads = [torch.empty_like(r) for _ in range(6)]
    dh0p = torch.empty_like(h0p)
    d_op = torch.randn(B * T, H, N, generator=gen).to(torch.bfloat16).to(dev)

    def packed_bwd():
        rc = lib.rwkv7_bwd_varlen(ptr(r), ptr(w), ptr(k), ptr(v), ptr(a), ptr(b), ptr(cu), n_seq, ptr(h0p),
                                  H * N * N, ptr(d_op), ptr(htp), *[ptr(g) for g in pgrads], ptr(dh0p),
                                  B * T, H, N, N, 0, ptr(pbws), pbws_bytes, stream)
        assert rc == 0, rc

    ms_packed_bwd, _ = time_gpu(packed_bwd, max(10, args.steps // 4), 3, torch)
    del pbws, pgrads, d_op, dh0p

    # ------------------------------------------------------------------ RWKV6 operator, the prefill shape
    u6 = a[0, 0].contiguous()                                   # [H, 64] bf16
    w6 = (w.float() * 2.0 - 1.0).to(torch.bfloat16)             # decays of about 0.70 .. 0.90 per step
    ws6_bytes = lib.rwkv6_fwd_workspace_bytes(B, T, H, 0)
    ws6 = torch.empty(ws6_bytes, dtype=torch.uint8, device=dev)

    def rwkv6():
        rc = lib.rwkv6_fwd(ptr(r), ptr(k), ptr(v), ptr(w6), ptr(u6), ptr(h0), B, None, ptr(o), ptr(ht),
                           B, T, H, N, N, 0, ptr(ws6), ws6_bytes, stream)
        assert rc == 0, rc

    ms_rwkv6, _ = time_gpu(rwkv6, args.steps, 3, torch)
    rwkv6_bytes = 5 * B * T * H * N * 2 + 2 * B * H * N * N * 4
    del ws6, w6

    # ------------------------------------------------------------------ one long sequence (few heads: two-kernel form)
    # BASELINE config 3: B=1, T=16384, H=64, zero initial state, the last 1024 tokens padded by the
    # w += (1 - mask) * -1e9 convention with r, k, v, a, b zeroed (the inputs of tests/test_gpu_fullsize.py)
    Bl, Tl, Hl, padl = 1, 16384, 64, 1024
    xl = list(make_inputs(Bl, Tl, Hl, N, seed=1237, dtype=torch.bfloat16, h0=False))
    maskl = torch.ones(Bl, Tl, 1, 1)
    maskl[:, Tl - padl:] = 0
    for i in (0, 2, 3, 4, 5):
        xl[i] = (xl[i].float() * maskl).to(torch.bfloat16)
    xl[1] = (xl[1].float() + (1 - maskl) * -1e9).to(torch.bfloat16)
    xl = [t.to(dev) for t in xl[:6]]
    ol = torch.empty_like(xl[0])
    htl = torch.empty(Bl, Hl, N, N, dtype=torch.float32, device=dev)
    wsl_bytes = lib.rwkv7_fwd_workspace_bytes(Bl, Tl, Hl, 0)
    wsl = torch.empty(wsl_bytes, dtype=torch.uint8, device=dev)

    def long_fwd():
        rc = lib.rwkv7_fwd(*[ptr(t) for t in xl[:6]], None, 0, ptr(ol), ptr(htl),
                           Bl, Tl, Hl, N, N, 0, ptr(wsl), wsl_bytes, stream)
        assert rc == 0, rc

    def long_summary():
        rc = lib.rwkv7_fwd_chunk_summary(*[ptr(t) for t in xl[:6]], Bl, Tl, Hl, N, N, 0, ptr(wsl), wsl_bytes, stream)
        assert rc == 0, rc

    def long_scan():
        rc = lib.rwkv7_fwd_chunk_scan(None, 0, ptr(ol), ptr(htl), Bl, Tl, Hl, N, N, 0,
                                      ptr(wsl), wsl_bytes, stream)
        assert rc == 0, rc

    ms_long, _ = time_gpu(long_fwd, args.steps, 3, torch)
    ms_long_summary, _ = time_gpu(long_summary, args.steps, 3, torch)
    ms_long_scan, _ = time_gpu(long_scan, args.steps, 3, torch)
    long_bytes = 7 * Bl * Tl * Hl * N * 2 + Bl * Hl * N * N * 4      # no initial state to read
    del wsl, xl, ol

    # ------------------------------------------------------------------ float32 inputs at the prefill shape
    # float32 callers get float32 arithmetic (1e-4 against the reference's native path): the recurrent kernel,
    # one token at a time with the state in registers
    x32 = [t.float() for t in (r, w, k, v, a, b)]
    o32 = torch.empty_like(x32[0])

    def fwd_f32():
        rc = lib.rwkv7_fwd(*[ptr(t) for t in x32], ptr(h0), H * N * N, ptr(o32), ptr(ht),
                           B, T, H, N, N, 1, None, 0, stream)
        assert rc == 0, rc

    ms_f32, _ = time_gpu(fwd_f32, max(5, args.steps // 10), 2, torch)
    f32_bytes = 7 * B * T * H * N * 4 + 2 * B * H * N * N * 4
    del x32, o32

    # float32 gradients at the training shape: the chunked float32 backward on the float32 matrix cores (rwkv7_bwd
    # with float32 tensors: the state before every 16-token chunk from one more forward pass, a chain kernel and a
    # per-chunk gradient kernel)
    xb32 = [t.float() for t in xb[:6]]
    d_o32 = d_o.float()
    g32 = [torch.empty_like(xb32[0]) for _ in range(6)]
    rws_bytes = lib.rwkv7_bwd_workspace_bytes(Bb, Tb, Hb, 1)
    rws = torch.empty(rws_bytes, dtype=torch.uint8, device=dev)

    def bwd_f32():
        rc = lib.rwkv7_bwd(*[ptr(t) for t in xb32], ptr(xb[6]), Hb * N * N, ptr(d_o32), ptr(d_ht),
                           *[ptr(g) for g in g32], ptr(dh0), Bb, Tb, Hb, N, N, 1, ptr(rws), rws_bytes, stream)
        assert rc == 0, rc

    ms_bwd_f32, _ = time_gpu(bwd_f32, max(5, args.steps // 10), 2, torch)
    # what the three kernels move per 16-token chunk and head: the forward pass 24 KiB in + 16 KiB state out, the
    # chain kernel 28 + 16 in and 16 (dh) + 8 (SA, dY) + 4 (dv) out, the gradient kernel 88 in and out
    bwd_f32_traffic = Bb * Hb * ((Tb + 15) // 16) * 200 * 1024
    del xb32, d_o32, g32, rws

    # ------------------------------------------------------------------ head size 128 (bf16, chunked forward)
    N2, B2, T2, H2 = 128, 8, 4096, 16                       # hidden 2048 as 16 heads of 128
    x128 = [t.to(dev) for t in make_inputs(B2, T2, H2, N2, seed=1240, dtype=torch.bfloat16)]
    o128 = torch.empty_like(x128[0])
    ht128 = torch.empty_like(x128[6])

    def fwd_128():
        rc = lib.rwkv7_fwd(*[ptr(t) for t in x128[:6]], ptr(x128[6]), H2 * N2 * N2, ptr(o128), ptr(ht128),
                           B2, T2, H2, N2, N2, 0, None, 0, stream)
        assert rc == 0, rc

    ms_128, _ = time_gpu(fwd_128, max(10, args.steps // 10), 2, torch)
    bytes_128 = 7 * B2 * T2 * H2 * N2 * 2 + 2 * B2 * H2 * N2 * N2 * 4
    # its gradients come from the float32 recurrent backward (there is no chunked backward for this head size):
    # a quarter of the sequence, on record as microseconds per token
    T3 = T2 // 4
    x128b = [t[:, :T3].contiguous() for t in x128[:6]]
    g128 = [torch.empty_like(x128b[0]) for _ in range(6)]
    dh128 = torch.empty_like(x128[6])
    ws128_bytes = lib.rwkv7_bwd_recurrent_workspace_bytes(B2, T3, H2, N2)
    ws128 = torch.empty(ws128_bytes, dtype=torch.uint8, device=dev)

    def bwd_128():
        rc = lib.rwkv7_bwd_recurrent(*[ptr(t) for t in x128b], ptr(x128[6]), H2 * N2 * N2, ptr(x128b[3]), ptr(ht128),
                                     *[ptr(g) for g in g128], ptr(dh128), B2, T3, H2, N2, N2, 0, ptr(ws128),
                                     ws128_bytes, stream)
        assert rc == 0, rc

    ms_128_bwd, _ = time_gpu(bwd_128, 3, 1, torch)
    del x128, o128, ht128, x128b, g128, dh128, ws128

    # ------------------------------------------------------------------ CPU baseline (rank 0, N = 1)
    cpu = None
    if not args.no_cpu:
        from oracle import rwkv7_native as orc
        threads = min(16, os.cpu_count() or 1)
        torch.set_num_threads(threads)
        # a bounded sample of the same workload: one of the 8 batch rows (all tokens, all heads),
        # float32 arithmetic on the bf16-rounded inputs (what the reference's native path does)
        Ts = T
        cx = [x[:1, :Ts].float() for x in xs[:6]] + [xs[6][:1]]
        orc.generalized_delta_rule(*[c[:, :32] for c in cx[:6]], cx[6])      # warm-up
        t0 = time.perf_counter()
        reps = 0
        while True:
            orc.generalized_delta_rule(*cx[:6], cx[6])
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 20:
                break
        dt = (time.perf_counter() - t0) / reps
        cpu = {"value": Ts / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
               "sample": f"B=1,T={Ts},H={H} slice of the step's inputs, torch restatement of the "
                         f"reference native loop (oracle/rwkv7_native.py), float32, {reps} reps, "
                         f"{dt:.2f} s each"}
        # the same slice through the C restatement (oracle/rwkv7_native.c, OpenMP over the heads)
        try:
            from oracle import native_c
            native_c.run(*[c[:, :32] for c in cx[:6]], cx[6])
            t0 = time.perf_counter()
            creps = 0
            while True:
                native_c.run(*cx[:6], cx[6])
                creps += 1
                if time.perf_counter() - t0 > 5.0 or creps >= 50:
                    break
            cdt = (time.perf_counter() - t0) / creps
            cpu["c_port"] = {"value": Ts / cdt, "unit": "tokens/s", "cores": min(H, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))),
                             "sample": f"same slice, oracle/rwkv7_native.c, float32, {creps} reps, {cdt:.3f} s each"}
        except Exception as exc:                                  # the C build is optional for the bench
            cpu["c_port"] = {"error": str(exc)}

        # BASELINE config 0 itself (B=1, T=256, H=4, float32, head_first=False, final state returned): the
        # reference's own CPU-runnable case on all host cores, one warm-up call and the median of five
        import statistics
        torch.set_num_threads(os.cpu_count() or 1)
        c0 = make_inputs(1, 256, 4, N, seed=1234, dtype=torch.float32)
        orc.generalized_delta_rule(*c0[:6], c0[6])
        times0 = []
        for _ in range(5):
            t0 = time.perf_counter()
            orc.generalized_delta_rule(*c0[:6], c0[6])
            times0.append(time.perf_counter() - t0)
        med0 = statistics.median(times0)
        cpu["config0"] = {"value": 256 / med0, "unit": "tokens/s", "cores": os.cpu_count() or 1,
                          "sample": f"B=1,T=256,H=4 float32 (BASELINE config 0), torch restatement of the reference "
                                    f"native loop, 1 warm-up + median of 5 calls, {med0 * 1e3:.1f} ms each"}
        torch.set_num_threads(threads)

    out = {
        "metric": "rwkv7_prefill_tokens_per_s",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "device_prewarm_steps": PREWARM_STEPS,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "chunked prefill generalized_delta_rule, B=8 T=4096 H=32 K=V=64, "
                               "bf16 r/w/k/v/a/b, float32 initial state in and final state out",
                   "global_batch": B, "seq_len": T, "heads": H, "head_size": N},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK, "traffic": MEASURED_TRAFFIC_BYTES,
                     "traffic_source": TRAFFIC_SOURCE,
                     "algorithmic_bytes": alg_bytes,
                     "kernel": "chunk_summary_kernel<MODE_FUSED> (one launch = one step)",
                     "kernel_ms": ms_fused,
                     "two_kernel_form": {"chunk_summary_kernel_ms": ms_summary, "chunk_scan_kernel_ms": ms_scan}},
        "mfma": {"algorithmic_tflops": alg_flops / (ms_step * 1e-3) / 1e12,
                 "algorithmic_frac_of_bf16_peak": alg_flops / (ms_step * 1e-3) / MFMA_BF16_PEAK,
                 "executed_flops_source": EXEC_FLOPS_SOURCE,
                 "executed_tflops": exec_flops / (ms_step * 1e-3) / 1e12,
                 "executed_frac_of_bf16_peak": exec_flops / (ms_step * 1e-3) / MFMA_BF16_PEAK},
        "decode": {"workload": f"T=1 decode, B={Bd} H={Hd}, bf16 inputs, float32 state updated in place, "
                               f"{nsteps} consecutive steps",
                   "us_per_step": us_per_decode_step, "state_GBps": dec_rate / 1e9,
                   "frac_of_hbm_peak": dec_rate / HBM_PEAK, "algorithmic_bytes_per_step": dec_bytes,
                   "no_reuse": {"workload": "same steps rotating over 4 states (672 MB > memory-side cache)",
                                "us_per_step": us_rot, "state_GBps": dec_bytes / (us_rot * 1e-6) / 1e9,
                                "frac_of_hbm_peak": dec_bytes / (us_rot * 1e-6) / HBM_PEAK}},
        "backward": {"workload": f"rwkv7_bwd (forward recomputed inside), B={Bb} T={Tb} H={Hb}, bf16, "
                                 "d_o and d_ht given, all seven gradients",
                     "ms": ms_bwd, "forward_ms_same_shape": ms_fwd_b,
                     "tokens_per_s": Bb * Tb / (ms_bwd * 1e-3), "algorithmic_bytes": bwd_bytes,
                     "algorithmic_GBps": bwd_bytes / (ms_bwd * 1e-3) / 1e9,
                     "frac_of_hbm_peak": bwd_bytes / (ms_bwd * 1e-3) / HBM_PEAK},
        "packed": {"workload": f"the step's {B * T} tokens as {n_seq} sequences of random lengths "
                               f"({min(y - x for x, y in zip(cu_host, cu_host[1:]))} .. "
                               f"{max(y - x for x, y in zip(cu_host, cu_host[1:]))}) in one packed row, H={H}, "
                               "per-sequence initial and final states (rwkv7_fwd_varlen / rwkv7_bwd_varlen)",
                   "forward_ms": ms_packed_fwd, "forward_tokens_per_s": B * T / (ms_packed_fwd * 1e-3),
                   "forward_frac_of_hbm_peak": (alg_bytes + 2 * (n_seq - B) * H * N * N * 4) / (ms_packed_fwd * 1e-3) / HBM_PEAK,
                   "backward_ms": ms_packed_bwd, "backward_tokens_per_s": B * T / (ms_packed_bwd * 1e-3)},
        "long_sequence": {"workload": f"BASELINE config 3: one sequence, B={Bl} T={Tl} H={Hl} bf16, zero initial state, the "
                                      f"last {padl} tokens masked by w += (1-mask)*-1e9 (rwkv7_fwd: per-chunk summaries, "
                                      "then the value-split scan, the form for fewer than 72 sequences)",
                          "ms": ms_long, "tokens_per_s": Bl * Tl / (ms_long * 1e-3),
                          "algorithmic_bytes": long_bytes,
                          "frac_of_hbm_peak": long_bytes / (ms_long * 1e-3) / HBM_PEAK,
                          "chunk_summary_kernel_ms": ms_long_summary, "chunk_scan_vsplit_kernel_ms": ms_long_scan,
                          "scan_us_per_chunk": ms_long_scan * 1e3 / (Tl // 64)},
        "float32": {"workload": f"generalized_delta_rule on float32 inputs, B={B} T={T} H={H} (the chunked float32 "
                                "kernel on the float32 matrix cores: 1e-4 parity with the reference's native path, "
                                "measured 3e-7)",
                    "ms": ms_f32, "tokens_per_s": B * T / (ms_f32 * 1e-3), "us_per_token": ms_f32 * 1e3 / T,
                    "algorithmic_bytes": f32_bytes, "frac_of_hbm_peak": f32_bytes / (ms_f32 * 1e-3) / HBM_PEAK,
                    # executed on the matrix cores per 16-token chunk and (batch, head): 4 x 80 instructions by the
                    # consumer waves, 96 by the producers, 2048 flops each (v_mfma_f32_16x16x4_f32)
                    "mfma_f32_executed_tflops": (B * H * ((T + 15) // 16) * 416 * 2048) / (ms_f32 * 1e-3) / 1e12,
                    "mfma_f32_frac_of_peak": (B * H * ((T + 15) // 16) * 416 * 2048) / (ms_f32 * 1e-3) / 157.3e12},
        "float32_backward": {"workload": f"rwkv7_bwd on float32 tensors (the chunked float32 backward on the float32 matrix "
                                         f"cores, forward states recomputed inside), B={Bb} T={Tb} H={Hb}, all seven gradients",
                             "ms": ms_bwd_f32, "us_per_token": ms_bwd_f32 * 1e3 / Tb,
                             "kernel_traffic_bytes": bwd_f32_traffic,
                             "kernel_traffic_frac_of_hbm_peak": bwd_f32_traffic / (ms_bwd_f32 * 1e-3) / HBM_PEAK},
        "head128": {"workload": f"rwkv7_fwd, K=V=128, B={B2} T={T2} H={H2} bf16 (the chunked kernel for that head size: one "
                                "workgroup per (batch, head), state in registers), float32 states in and out",
                    "ms": ms_128, "tokens_per_s": B2 * T2 / (ms_128 * 1e-3), "us_per_chunk": ms_128 * 1e3 / (T2 // 64),
                    "algorithmic_bytes": bytes_128, "frac_of_hbm_peak": bytes_128 / (ms_128 * 1e-3) / HBM_PEAK,
                    "backward": {"workload": f"rwkv7_bwd_recurrent, K=V=128, B={B2} T={T3} H={H2} bf16 (token by token in "
                                             "float32: this head size has no chunked backward)",
                                 "ms": ms_128_bwd, "us_per_token": ms_128_bwd * 1e3 / T3}},
        "rwkv6": {"workload": f"RWKV6 operator forward (rwkv6_fwd), B={B} T={T} H={H} bf16, float32 states in and out",
                  "ms": ms_rwkv6, "tokens_per_s": B * T / (ms_rwkv6 * 1e-3), "algorithmic_bytes": rwkv6_bytes,
                  "frac_of_hbm_peak": rwkv6_bytes / (ms_rwkv6 * 1e-3) / HBM_PEAK},
        "cpu_baseline": cpu,
        "build": {"library": os.path.relpath(_lib.LIB_PATH, ROOT), "library_sha256_16": file_digest(_lib.LIB_PATH),
                  "abi_version": int(lib.rwkv7_abi_version()), "sources_sha256_16": sources_digest(),
                  "profile_constants_taken_at_sources_sha256_16": CONSTANTS_SOURCES_DIGEST,
                  "profile_constants_current": sources_digest() == CONSTANTS_SOURCES_DIGEST},
        "wall_ms_per_step": wall_ms,
        "device": props.name,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
