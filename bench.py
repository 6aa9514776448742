#!/usr/bin/env python3
"""Benchmark of the GGUF k-quant decode path on one MI355X.

    python bench.py [--gpus 1] [--steps 128] [--warmup 8]

A "step" is one greedy decode token of the Qwen3-4B-shaped Q4_K_M model (36 layers, hidden 2560,
32 q / 8 kv heads, head_dim 128, ffn 9728, vocab 151936; random-init seeded super-blocks; fp16 KV
cache prefilled with 2048 seeded positions), i.e. BASELINE.json configs[3].  Weights, KV cache and
scratch are resident in HBM before the timed region starts.  One JSON line is printed on stdout.

Besides the token rate the line carries
  roofline      the kernel that costs most per token - of the fused RMSNorm + Q4_K gate/up GEMV + SiLU (2 x 9728 x 2560)
                and the Q6_K down projection (2560 x 9728), both reported under roofline.kernels: algorithmic bytes per
                launch / average launch duration measured with HIP events on the launching stream, cycling over the
                36 layers' distinct weights; traffic from the rocprofv3 counter summary under profiles/
  gemv          the same measurement for configs[0] (Q4_K 9728x2560) and configs[1] (Q6_K lm_head)
  cpu_baseline  the reference's CPU path (oracle/_ref build if present, else this repo's C port)
                timed on this host for a bounded number of tokens of the same workload
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "decode_qwen3_4b_hbm_traffic_pmc.md")
SEED = 25
N_PREFILL = 2048
MAX_SEQ = 2304


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def measured_traffic():
    """HBM bytes per launch of the decode kernels, as the rocprofv3 FETCH_SIZE / WRITE_SIZE summary under profiles/ records
    them: its lines `TRAFFIC <kernel key> fetch_kib=<..> write_kib=<..>` (KiB per dispatch), `FETCH_SCALE <factor>` (what
    FETCH_SIZE reads for a copy of known size) and `MEASURED_AT <commit>`.  Returns ({key: bytes}, commit) or ({}, None)."""
    import re
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return {}, None
    scale = re.search(r"^FETCH_SCALE\s+([0-9.]+)", text, re.M)
    commit = re.search(r"^MEASURED_AT\s+(\S+)", text, re.M)
    out = {}
    for key, f, w in re.findall(r"^TRAFFIC\s+(\S+)\s+fetch_kib=([0-9.]+)\s+write_kib=([0-9.]+)", text, re.M):
        out[key] = int((float(f) * float(scale.group(1) if scale else 1.0) + float(w)) * 1024)
    return out, (commit.group(1) if commit else None)


def bench_lib():
    """libptm_bench.so (bench_kernels.hip): the streaming-read kernel used as the achievable ceiling; not part of the product
    library."""
    import ctypes as C
    path = os.path.join(ROOT, "libptm_bench.so")
    if not os.path.exists(path):
        raise ImportError(path + " is not built: python -c 'import __graft_entry__ as g; g.build()'")
    L = C.CDLL(path)
    L.bench_stream_read_partials.restype = C.c_int64
    L.bench_stream_read_partials.argtypes = [C.c_int64]
    L.bench_stream_read_xor.restype = C.c_int
    L.bench_stream_read_xor.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]
    return L


def event_time_ms(fn, iters, torch):
    """Average GPU duration of fn(i) over `iters` launches: the launches are captured into one graph
    (so the host's per-call cost does not throttle them) and a replay is bracketed by HIP events
    recorded on the stream the kernels run on; the median of three replays (a single short replay can
    fall into a clock transient)."""
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        for i in range(4):
            fn(i)  # first calls outside capture (one-time kernel attributes)
        st.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            for i in range(iters):
                fn(i)
        g.replay()
        st.synchronize()
        times = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(st)
            g.replay()
            e1.record(st)
            st.synchronize()
            times.append(e0.elapsed_time(e1))
    return sorted(times)[1] / iters


def only_kernel(which, torch, ops, synth):
    """One prompt-pass kernel by itself, for counter passes: the cfg4 gate-projection GEMM (512 x 4096 x 14336, Q4_K) or the
    causal attention of 512 / 2048 prompt rows at the Qwen3-4B head shape."""
    def timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3
    if which == "prefill_gemm":
        M, K, N = 512, 4096, 14336
        W = torch.from_numpy(synth.make_q4k(synth.rng_for(SEED, 5), N, K)).cuda()
        X = torch.randn(M, K, device="cuda").to(torch.bfloat16)
        Y = torch.empty(M, N, device="cuda")
        ws = torch.empty(ops.qgemm_f16_workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
        us = timed(lambda: ops.matmul_q_f16(12, W, X, Y, M, K, N, K // 256 * 144, ws), 6)
        return {"only": which, "shape": [M, K, N], "us_with_row_conversion": us}
    nh, nkv, hd, max_seq = 32, 8, 128, 2304
    Kc = torch.randn(max_seq, nkv * hd, device="cuda").half()
    Vc = torch.randn(max_seq, nkv * hd, device="cuda").half()
    out = {"only": which}
    for rows in (512, 2048):
        Q = torch.randn(rows, nh * hd, device="cuda")
        O = torch.empty_like(Q)
        out["us_%d_rows" % rows] = timed(lambda: ops.prefill_attention(Q, Kc, Vc, O, rows, nh, nkv, hd, 0, max_seq, hd ** -0.5, True), 6)
    return out


def main():
    # stdout carries exactly one line, the JSON result: anything a native library prints to file descriptor 1 in the
    # meantime (the compiled reference reports its scratch allocation there) is sent to stderr instead
    sys.stdout.flush()
    json_fd = os.dup(1)
    os.dup2(2, 1)
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--cpu-tokens", type=int, default=16, help="tokens of the CPU baseline sample (0 = skip)")
    ap.add_argument("--cpu-child", type=int, default=0, help=argparse.SUPPRESS)  # the 1-thread CPU measurement, see cpu_child_main
    ap.add_argument("--long-context", type=int, default=1, help="0: skip the decode measurements at 8192 / 32768 positions")
    ap.add_argument("--mix-steps", type=int, default=64, help="decode steps of the alternating Q4_K / Q6_K type mix (0 = skip)")
    ap.add_argument("--gemma-steps", type=int, default=64,
                    help="decode steps of the Gemma-3-4B-shaped extra (0: skip it)")
    ap.add_argument("--qwen25-steps", type=int, default=64, help="decode steps of the Qwen2.5-7B-shaped model (0 = skip)")
    ap.add_argument("--llama-steps", type=int, default=64,
                    help="decode steps of the Llama-3-8B-shaped extra measurement (0 = skip)")
    ap.add_argument("--layers", type=int, default=36, help=argparse.SUPPRESS)  # debugging only; 36 is the workload
    ap.add_argument("--only", choices=["prefill_gemm", "prefill_attention"], default=None,
                    help="launch just this prompt-pass kernel a few times and print its time: the target of the counter "
                         "passes behind the figures quoted for it (rocprofv3 --pmc ... -- python3 bench.py --only ...)")
    args = ap.parse_args()
    if args.cpu_child > 0:
        os.dup2(json_fd, 1)
        cpu_child_main(args.cpu_child)
        return
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU (batch-1 decode); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if args.steps + args.warmup + N_PREFILL + 1 > MAX_SEQ:
        print("bench.py: steps + warmup must stay below %d" % (MAX_SEQ - N_PREFILL - 1), file=sys.stderr)
        sys.exit(2)

    # the 1-thread CPU baseline runs beside everything below, in a child started before this process touches the GPU
    child = None
    if args.cpu_tokens > 0 and not args.only:
        import subprocess
        env = dict(os.environ, PT_NUM_THREADS="1", OMP_NUM_THREADS="1")
        child = subprocess.Popen([sys.executable, os.path.abspath(__file__), "--cpu-child", str(args.cpu_tokens)],
                                 stdout=subprocess.PIPE, env=env)

    import torch
    from prometorch_amd import _lib, ops
    from prometorch_amd.testing import synth
    from prometorch_amd.decode import Decoder

    _lib.load()  # fails loudly when the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    if args.only:
        os.write(json_fd, (json.dumps(only_kernel(args.only, torch, ops, synth)) + "\n").encode())
        return
    baseline = json.load(open(os.path.join(ROOT, "BASELINE.json")))

    cfg = dict(synth.QWEN3_4B)
    cfg["n_layers"] = args.layers
    t0 = time.time()
    layers = [synth.make_layer(SEED, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(SEED, cfg)
    log("synthetic model generated in %.1fs" % (time.time() - t0))
    dec = Decoder(cfg, layers, head, max_seq=MAX_SEQ, kv_fp16=True, use_graph=True)
    kvs = []
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEED, i, cfg, N_PREFILL)
        dec.set_kv(i, k, v)
        kvs.append((k, v))
    torch.cuda.synchronize()
    log("uploaded in %.1fs" % (time.time() - t0))

    # The host loops below are timed per token; a full collection of the interpreter's object graph (tens of
    # milliseconds once torch is imported) landing inside one of them would be charged to that loop
    import gc
    gc.collect()
    gc.disable()

    # ---- timed region: W warm-up tokens, then exactly K tokens, host-synchronous per token ----
    dec.set_past_len(N_PREFILL)
    tok = 1
    for _ in range(args.warmup):
        tok = dec.step(tok)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    toks = []
    for _ in range(args.steps):
        tok = dec.step(tok)
        toks.append(tok)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t1
    tok_s = args.steps / dt
    log("decode: %d tokens in %.4fs = %.1f tok/s (%.3f ms/token)" % (args.steps, dt, tok_s, dt / args.steps * 1e3))

    # same tokens with device-side token feedback (no host round trip between tokens)
    dec.set_past_len(N_PREFILL)
    dec.greedy(1, args.warmup)
    t1 = time.perf_counter()
    dec.set_past_len(N_PREFILL)
    chained = dec.greedy(1, args.warmup + args.steps)
    dt_chain = time.perf_counter() - t1
    chained_tok_s = (args.warmup + args.steps) / dt_chain
    tokens_equal = chained[args.warmup:] == toks
    log("chained: %.1f tok/s, tokens identical to stepwise: %s" % (chained_tok_s, tokens_equal))

    # sampled generation with the sampler on the device (temperature 0.8, top-k 40, top-p 0.9, repetition penalty 1.1:
    # PromeServe's defaults), host-synchronous per token like the timed greedy loop, and chained
    us = ops.mt19937_uniforms(42, 0, args.warmup + args.steps)
    dec.set_past_len(N_PREFILL)
    dec.sampling_begin(0.8, 40, 0.9, 1.1)
    tok_s_ = 1
    for i in range(args.warmup):
        tok_s_ = dec.sample(tok_s_, us[i:i + 1])[0]
    t1 = time.perf_counter()
    for i in range(args.steps):
        tok_s_ = dec.sample(tok_s_, us[args.warmup + i:args.warmup + i + 1])[0]
    sampled_tok_s = args.steps / (time.perf_counter() - t1)
    dec.set_past_len(N_PREFILL)
    dec.sampling_begin(0.8, 40, 0.9, 1.1)
    t1 = time.perf_counter()
    dec.sample(1, us)
    sampled_chained_tok_s = (args.warmup + args.steps) / (time.perf_counter() - t1)
    log("sampled (device top-k/top-p): %.1f tok/s per-token sync, %.1f tok/s chained" % (sampled_tok_s, sampled_chained_tok_s))
    gc.enable()

    # ---- roofline of the dominant kernel, live, HIP events on the launching stream --------------
    H, I = cfg["hidden"], cfg["inter"]
    L0 = dec._layers
    nL = cfg["n_layers"]
    x = torch.randn(H, device="cuda")
    act = torch.empty(I, device="cuda")
    stride4 = H // 256 * 144
    gate_up_bytes = 2 * I * stride4 + 4 * H + 4 * H + 4 * I  # two matrices + x + gamma in, act out

    def run_gate_up(i):
        Ld = L0[i % nL]
        ops.fused_rmsnorm_gate_up_silu(x, Ld.ffn_norm, Ld.gate.data, Ld.up.data, act, H, I, stride4, 1e-6, False)

    ms = event_time_ms(run_gate_up, 360, torch)
    log("gate/up fused: %.2f us/launch, %.0f GB/s" % (ms * 1e3, gate_up_bytes / (ms * 1e-3) / 1e9))

    gemv = {}
    # configs[0]: single Q4_K GEMV 9728x2560 (x quantised in the kernel), cold (36 distinct matrices) and warm
    y = torch.empty(I, device="cuda")
    b0 = I * stride4 + 4 * H + 4 * I
    ms_cold = event_time_ms(lambda i: ops.launch_q4km_persistent_gemv(L0[i % nL].gate.data, x, y, H, I, stride4), 360, torch)
    ms_warm = event_time_ms(lambda i: ops.launch_q4km_persistent_gemv(L0[0].gate.data, x, y, H, I, stride4), 360, torch)
    gemv["cfg0_q4k_9728x2560"] = {"bytes": b0, "us_cold": ms_cold * 1e3, "GBs_cold": b0 / ms_cold / 1e6,
                                  "frac_cold": b0 / ms_cold / 1e6 / HBM_PEAK_GBS, "us_warm_cache": ms_warm * 1e3,
                                  "GBs_warm_cache": b0 / ms_warm / 1e6}
    # configs[1]: Q6_K lm_head 151936x2560 + argmax
    V = cfg["vocab"]
    stride6 = H // 256 * 210
    logits = torch.empty(V, device="cuda")
    idx = torch.zeros(1, dtype=torch.int64, device="cuda")
    ws = torch.empty(ops.argmax_workspace_bytes(V), dtype=torch.uint8, device="cuda")
    b1 = V * stride6 + 4 * H + 4 * V
    lm = dec._cfg.lm_head.data
    ms1 = event_time_ms(lambda i: ops.q6k_gemv_argmax(lm, x, logits, H, V, stride6, idx, ws), 40, torch)
    gemv["cfg1_q6k_lm_head_argmax"] = {"bytes": b1, "us": ms1 * 1e3, "GBs": b1 / ms1 / 1e6, "frac": b1 / ms1 / 1e6 / HBM_PEAK_GBS}
    # the GEMV launch by itself (logits only): the op above is this launch with per-workgroup argmax partials plus the
    # one-workgroup launch that finishes the argmax
    ms1g = event_time_ms(lambda i: ops.launch_q6k_gemv(lm, x, logits, H, V, stride6), 40, torch)
    gemv["cfg1_q6k_lm_head_argmax"].update({"us_gemv_launch": ms1g * 1e3, "GBs_gemv_launch": b1 / ms1g / 1e6,
                                            "frac_gemv_launch": b1 / ms1g / 1e6 / HBM_PEAK_GBS})
    # the Q4_K kernel on a launch large enough to amortise the launch floor (vocabulary-sized, 219 MB): shows what
    # the kernel sustains once the ~1.6 us launch + ramp no longer dominates, as it does for a 14 MB matrix
    Wbig = [torch.from_numpy(synth.make_q4k(synth.rng_for(SEED, 6 + i), V, H)).cuda() for i in range(3)]  # 657 MB > caches
    ybig = torch.empty(V, device="cuda")
    b3 = V * stride4 + 4 * H + 4 * V
    ms3 = event_time_ms(lambda i: ops.launch_q4km_persistent_gemv(Wbig[i % 3], x, ybig, H, V, stride4), 42, torch)
    gemv["q4k_large_151936x2560"] = {"bytes": b3, "us": ms3 * 1e3, "GBs": b3 / ms3 / 1e6, "frac": b3 / ms3 / 1e6 / HBM_PEAK_GBS}
    del Wbig, ybig
    # down projection Q6_K 2560x9728
    xa = torch.randn(I, device="cuda")
    yd = torch.zeros(H, device="cuda")
    strided = I // 256 * 210
    b2 = H * strided + 4 * I + 4 * H
    ms2 = event_time_ms(lambda i: ops.launch_q6k_gemv(L0[i % nL].down.data, xa, yd, I, H, strided, accumulate=True), 360, torch)
    gemv["q6k_down_2560x9728"] = {"bytes": b2, "us": ms2 * 1e3, "GBs": b2 / ms2 / 1e6, "frac": b2 / ms2 / 1e6 / HBM_PEAK_GBS}
    # The two GEMV kernels that share the top of the per-token budget (36 launches each): fused RMSNorm + Q4_K gate/up + SiLU
    # and the Q6_K down projection accumulating into the residual.  `roofline` is the one that costs more per token.
    traffic, traffic_commit = measured_traffic()
    kernels = {
        "gate_up": {"kernel": "q4k_gemv_kernel<fused rmsnorm + gate/up + silu> 2x9728x2560", "bytes_per_launch": gate_up_bytes,
                    "us_per_launch": ms * 1e3, "launches_per_token": nL},
        "down": {"kernel": "q6k_gemv_tall_kernel<accumulate> 2560x9728", "bytes_per_launch": b2, "us_per_launch": ms2 * 1e3,
                 "launches_per_token": nL},
    }
    for key, kq in kernels.items():
        kq["achieved"] = kq["bytes_per_launch"] / kq["us_per_launch"] / 1e3
        kq["frac"] = kq["achieved"] / HBM_PEAK_GBS
        kq["traffic"] = traffic.get(key) if args.layers == 36 else None
    dom = max(kernels, key=lambda k: kernels[k]["us_per_launch"] * kernels[k]["launches_per_token"])
    roof = {"bound": "hbm", "kernel": kernels[dom]["kernel"], "achieved": kernels[dom]["achieved"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": kernels[dom]["frac"], "traffic": kernels[dom]["traffic"],
            "bytes_per_launch": kernels[dom]["bytes_per_launch"], "us_per_launch": kernels[dom]["us_per_launch"],
            "traffic_measured_at": traffic_commit, "kernels": kernels}
    # configs[4] (prefill): Llama-3-8B gate projection 14336x4096 (Q4_K), 512 bf16 rows, both GEMM kernels
    Mq, Kq, Nq = 512, 4096, 14336
    Wq = torch.from_numpy(synth.make_q4k(synth.rng_for(SEED, 5), Nq, Kq)).cuda()
    Xq = torch.randn(Mq, Kq, device="cuda").to(torch.bfloat16)
    Yq = torch.empty(Mq, Nq, device="cuda")
    wsq = torch.empty(max(ops.qgemm_workspace_bytes(Mq, Kq), ops.qgemm_f16_workspace_bytes(Mq, Kq)), dtype=torch.uint8, device="cuda")
    flop = 2.0 * Mq * Kq * Nq
    # 100 launches per replay: shorter bursts of this matrix-core kernel are timed during the clock ramp (85-95 us against 78)
    msf = event_time_ms(lambda i: ops.matmul_q_f16(12, Wq, Xq, Yq, Mq, Kq, Nq, Kq // 256 * 144, wsq), 100, torch)
    gemv["cfg4_q4k_prefill_gemm_512x4096x14336_f16_mfma"] = {
        "flop": flop, "us": msf * 1e3, "TFLOPs": flop / msf / 1e9, "frac_f16_mfma_peak": flop / msf / 1e9 / 2500.0,
        "numerics": "Q8-rounded activations and dequantised weights in fp16, fp32 accumulate; within 5e-3 of rms(y) of the reference GEMV per row"}
    msq = event_time_ms(lambda i: ops.matmul_q(12, Wq, Xq, Yq, Mq, Kq, Nq, Kq // 256 * 144, wsq), 40, torch)
    gemv["cfg4_q4k_prefill_gemm_512x4096x14336_int8_mfma_exact"] = {
        "ops": flop, "us": msq * 1e3, "TOPs": flop / msq / 1e9, "frac_int8_mfma_peak": flop / msq / 1e9 / 5000.0,
        "numerics": "rows bit-identical to the reference GEMV"}
    del Wq, Xq, Yq, wsq
    # plain copy of known size: the kernel the HBM byte counters are scaled by
    ca = torch.empty(64 << 20, device="cuda")
    cb = torch.empty(64 << 20, device="cuda")
    msc = event_time_ms(lambda i: ops.launch_copy(ca, cb, ca.numel()), 4, torch)
    gemv["copy_256MiB"] = {"bytes_read": ca.numel() * 4, "bytes_written": ca.numel() * 4, "us": msc * 1e3,
                           "GBs": 2 * ca.numel() * 4 / msc / 1e6}
    del ca, cb
    # pure streaming reads of the GEMV footprints (cold: 36 distinct spans of a 1 GB buffer; the lm_head once per launch):
    # the ceiling that launches of this size can reach on this part, beside the nominal 8 TB/s
    span = 2 * I * stride4
    pool = torch.empty(36 * span, dtype=torch.uint8, device="cuda")
    BL = bench_lib()
    parts = torch.empty(BL.bench_stream_read_partials(V * stride6), dtype=torch.int32, device="cuda")

    def stream_read(ptr, nb):
        rc = BL.bench_stream_read_xor(ptr, nb, parts.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    ceil = {}
    for name, nb in (("14MB_one_q4k_matrix", I * stride4), ("20MB_q6k_down", H * strided), ("28MB_gate_up", span)):
        msr = event_time_ms(lambda i: stream_read(pool[(i % 36) * span:].data_ptr(), nb), 360, torch)
        ceil[name] = {"bytes": nb, "us": msr * 1e3, "GBs": nb / msr / 1e6}
    msr = event_time_ms(lambda i: stream_read(lm, V * stride6), 40, torch)
    ceil["319MB_lm_head"] = {"bytes": V * stride6, "us": msr * 1e3, "GBs": V * stride6 / msr / 1e6}
    gemv["stream_read_ceiling"] = ceil
    kernels["gate_up"]["frac_of_stream_read"] = kernels["gate_up"]["achieved"] / ceil["28MB_gate_up"]["GBs"]
    kernels["down"]["frac_of_stream_read"] = kernels["down"]["achieved"] / ceil["20MB_q6k_down"]["GBs"]
    roof["frac_of_stream_read"] = kernels[dom]["frac_of_stream_read"]
    log("stream-read ceiling: " + ", ".join("%s %.2f us" % (k, v["us"]) for k, v in ceil.items()))
    del pool, parts
    # prompt prefill through all layers: 512 tokens from an empty context (row-batched GEMMs + causal attention)
    prompt = [int(t) for t in synth.rng_for(SEED, 9).integers(0, V, 512)]
    layer_params = H * (2 * cfg["n_heads"] * cfg["head_dim"] + 2 * cfg["n_kv_heads"] * cfg["head_dim"] + 3 * I)
    dec.set_past_len(0)
    dec.prefill(prompt)  # allocates the row scratch
    t1 = time.perf_counter()
    for _ in range(3):
        dec.set_past_len(0)
        dec.prefill(prompt)
    dtp = (time.perf_counter() - t1) / 3
    gemv["prefill_512_tokens"] = {"ms": dtp * 1e3, "tok_s": 512 / dtp,
                                  "gemm_TFLOPs": 2.0 * 512 * nL * layer_params / dtp / 1e12}
    prompt2k = [int(t) for t in synth.rng_for(SEED, 10).integers(0, V, 2048)]
    dec.set_past_len(0)
    dec.prefill(prompt2k)  # grows the row scratch to 2048 rows
    t1 = time.perf_counter()
    for _ in range(2):
        dec.set_past_len(0)
        dec.prefill(prompt2k)
    dtp = (time.perf_counter() - t1) / 2
    gemv["prefill_2048_tokens"] = {"ms": dtp * 1e3, "tok_s": 2048 / dtp,
                                   "gemm_TFLOPs": 2.0 * 2048 * nL * layer_params / dtp / 1e12}
    log(json.dumps(gemv))
    per_token_bytes = nL * 63866880 + V * stride6 + nL * 2 * (N_PREFILL + args.warmup + args.steps / 2) * 1024 * 2
    dec.close()
    del dec
    torch.cuda.empty_cache()

    # ---- a second model family on the same decoder: Llama-3-8B-shaped Q4_K_M (no QK-norm, interleaved rotation) -----
    llama = None
    if args.llama_steps > 0:
        t0 = time.perf_counter()
        lcfg = dict(synth.LLAMA3_8B)
        _, llayers, lhead = synth.llama3_8b_like(SEED + 1, n_layers=lcfg["n_layers"], vocab=lcfg["vocab"])
        ldec = Decoder(lcfg, llayers, lhead, max_seq=MAX_SEQ, kv_fp16=True, use_graph=True)
        for i in range(lcfg["n_layers"]):
            ldec.set_kv(i, *synth.make_kv_prefill(SEED + 1, i, lcfg, N_PREFILL))
        ldec.set_past_len(N_PREFILL)
        ltok = 1
        for _ in range(args.warmup):
            ltok = ldec.step(ltok)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.llama_steps):
            ltok = ldec.step(ltok)
        torch.cuda.synchronize()
        ldt = time.perf_counter() - t1
        llama = {"workload": "batch-1 greedy decode, Llama-3-8B-shaped Q4_K_M (32 layers, 4096 hidden, 14336 intermediate, "
                             "128256 vocabulary), fp16 KV prefilled %d, %d new tokens, host-synchronous" % (N_PREFILL, args.llama_steps),
                 "tok_s": args.llama_steps / ldt, "ms_per_token": ldt / args.llama_steps * 1e3,
                 "token_hbm_frac": (32 * 138_903_552 + 128256 * 3360 + 32 * 2 * (N_PREFILL + args.warmup + args.llama_steps / 2) * 1024 * 2)
                                   / (ldt / args.llama_steps) / 1e9 / HBM_PEAK_GBS,
                 "a100_published_deepseek_r1_8b_tok_s": 51.1}
        log("llama-3-8B shape: %.1f tok/s (%.3f ms/token), set up in %.1fs" % (llama["tok_s"], llama["ms_per_token"], t1 - t0))
        ldec.close()
        del ldec, llayers, lhead
        torch.cuda.empty_cache()

    # ---- the 7B size: Qwen2.5-7B-shaped Q4_K_M (7 query heads per kv head, q / k / v biases, no QK-norm; rows of 14 and 74
    # super-blocks: the down projection 3584 x 18944 is the widest few-long-rows launch of the families here) -----------------
    q25 = None
    if args.qwen25_steps > 0:
        t0 = time.perf_counter()
        qcfg = dict(synth.QWEN25_7B)
        _, qlayers, qhead = synth.qwen25_7b_like(SEED + 3, n_layers=qcfg["n_layers"], vocab=qcfg["vocab"])
        qdec = Decoder(qcfg, qlayers, qhead, max_seq=MAX_SEQ, kv_fp16=True, use_graph=True)
        for i in range(qcfg["n_layers"]):
            qdec.set_kv(i, *synth.make_kv_prefill(SEED + 3, i, qcfg, N_PREFILL))
        qdec.set_past_len(N_PREFILL)
        qtok = 1
        for _ in range(args.warmup):
            qtok = qdec.step(qtok)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.qwen25_steps):
            qtok = qdec.step(qtok)
        torch.cuda.synchronize()
        qdt = time.perf_counter() - t1
        qH, qI, qV = qcfg["hidden"], qcfg["inter"], qcfg["vocab"]
        qqd, qkvd = qcfg["n_heads"] * qcfg["head_dim"], qcfg["n_kv_heads"] * qcfg["head_dim"]
        q_layer = (qqd * qH + qkvd * qH + qH * qqd + 2 * qI * qH) // 256 * 144 + (qkvd * qH + qH * qI) // 256 * 210
        q_bytes = qcfg["n_layers"] * (q_layer + 2 * (N_PREFILL + args.warmup + args.qwen25_steps / 2) * qkvd * 2) + qV * (qH // 256 * 210)
        q25 = {"workload": "batch-1 greedy decode, Qwen2.5-7B-shaped Q4_K_M (%d layers, %d hidden, %d x 128 heads on %d kv heads, "
                           "%d intermediate, %d vocabulary, q / k / v biases), fp16 KV prefilled %d, %d new tokens, host-synchronous"
                           % (qcfg["n_layers"], qH, qcfg["n_heads"], qcfg["n_kv_heads"], qI, qV, N_PREFILL, args.qwen25_steps),
               "tok_s": args.qwen25_steps / qdt, "ms_per_token": qdt / args.qwen25_steps * 1e3,
               "token_hbm_frac": q_bytes / (qdt / args.qwen25_steps) / 1e9 / HBM_PEAK_GBS}
        log("qwen2.5-7B shape: %.1f tok/s (%.3f ms/token), set up in %.1fs" % (q25["tok_s"], q25["ms_per_token"], t1 - t0))
        qdec.close()
        del qdec, qlayers, qhead
        torch.cuda.empty_cache()

    # ---- a third family: Gemma-3-4B-shaped Q4_K_M (256-wide heads, post-norms, GELU gate, sliding-window layers) ----
    gemma = None
    if args.gemma_steps > 0:
        t0 = time.perf_counter()
        gcfg = dict(synth.GEMMA3_4B)
        _, glayers, ghead = synth.gemma3_4b_like(SEED + 2, n_layers=gcfg["n_layers"], vocab=gcfg["vocab"])
        gdec = Decoder(gcfg, glayers, ghead, max_seq=MAX_SEQ, kv_fp16=True, use_graph=True)
        for i in range(gcfg["n_layers"]):
            gdec.set_kv(i, *synth.make_kv_prefill(SEED + 2, i, gcfg, N_PREFILL))
        gdec.set_past_len(N_PREFILL)
        gtok = 1
        for _ in range(args.warmup):
            gtok = gdec.step(gtok)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.gemma_steps):
            gtok = gdec.step(gtok)
        torch.cuda.synchronize()
        gdt = time.perf_counter() - t1
        g_T = N_PREFILL + args.warmup + args.gemma_steps / 2
        g_bytes = 34 * 60_518_400 + 262144 * 2100 + 2 * (29 * 1024 + 5 * g_T) * 1024 * 2
        gemma = {"workload": "batch-1 greedy decode, Gemma-3-4B-shaped Q4_K_M (34 layers, 2560 hidden, 8 x 256 heads on 4 kv heads, "
                             "10240 intermediate, 262144 vocabulary, window 1024 on 29 layers), fp16 KV prefilled %d, %d new tokens, "
                             "host-synchronous" % (N_PREFILL, args.gemma_steps),
                 "tok_s": args.gemma_steps / gdt, "ms_per_token": gdt / args.gemma_steps * 1e3,
                 "token_hbm_frac": g_bytes / (gdt / args.gemma_steps) / 1e9 / HBM_PEAK_GBS,
                 "a100_published_gemma3_4b_tok_s": 81.4}
        gprompt = [int(t) for t in synth.rng_for(SEED + 2, 9).integers(0, gcfg["vocab"], 512)]
        gdec.set_past_len(0)
        gdec.prefill(gprompt)  # allocates the row scratch
        t2 = time.perf_counter()
        for _ in range(3):
            gdec.set_past_len(0)
            gdec.prefill(gprompt)
        gemma["prefill_512_tokens_ms"] = (time.perf_counter() - t2) / 3 * 1e3
        log("gemma-3-4B shape: %.1f tok/s (%.3f ms/token), 512-token prompt %.2f ms, set up in %.1fs"
            % (gemma["tok_s"], gemma["ms_per_token"], gemma["prefill_512_tokens_ms"], t1 - t0))
        gdec.close()
        del gdec, glayers, ghead
        torch.cuda.empty_cache()

    # ---- what real Q4_K_M files look like: attn_v and ffn_down alternate between Q6_K and Q4_K from layer to layer
    # (Q6_K in the first and the last eighth of the layers and in every third layer between, Q4_K elsewhere: the rule the
    # reference's loader meets in such files, cpu_quant_gemv.h:1458-1460) -----------------------------------------------
    mix = None
    if args.mix_steps > 0:
        nLm = cfg["n_layers"]

        def more_bits(li):
            return li < nLm // 8 or li >= 7 * nLm // 8 or (li - nLm // 8) % 3 == 2

        mlayers = []
        for li in range(nLm):
            t = 14 if more_bits(li) else 12
            mats = tuple((n, t if n in ("v", "down") else q) for n, q in synth.LAYER_MATS)
            mlayers.append(layers[li] if t == 14 else synth.make_layer(SEED, li, cfg, mats=mats))
        n_q6 = sum(1 for li in range(nLm) if more_bits(li))
        mdec = Decoder(cfg, mlayers, head, max_seq=MAX_SEQ, kv_fp16=True, use_graph=True)
        for i in range(nLm):
            mdec.set_kv(i, *kvs[i])
        mdec.set_past_len(N_PREFILL)
        mtok = 1
        for _ in range(args.warmup):
            mtok = mdec.step(mtok)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.mix_steps):
            mtok = mdec.step(mtok)
        torch.cuda.synchronize()
        mdt = time.perf_counter() - t1
        # the Q4_K down projection 2560 x 9728 (accumulating), cycling the layers that hold one
        q4_layers = [i for i in range(nLm) if not more_bits(i)]
        xa4 = torch.randn(I, device="cuda")
        yd4 = torch.zeros(H, device="cuda")
        sd4 = I // 256 * 144
        bd4 = H * sd4 + 4 * I + 4 * H
        ML = mdec._layers
        msd4 = event_time_ms(lambda i: ops.launch_q4km_persistent_gemv_accumulate(ML[q4_layers[i % len(q4_layers)]].down.data, xa4, yd4, I, H, sd4),
                             360, torch)
        mix = {"workload": "batch-1 greedy decode, Qwen3-4B shape with the attn_v / ffn_down types of a Q4_K_M file: Q6_K in %d layers, "
                           "Q4_K in %d; fp16 KV prefilled %d, %d new tokens, host-synchronous" % (n_q6, nLm - n_q6, N_PREFILL, args.mix_steps),
               "tok_s": args.mix_steps / mdt, "ms_per_token": mdt / args.mix_steps * 1e3,
               "q4k_down_2560x9728": {"bytes": bd4, "us": msd4 * 1e3, "GBs": bd4 / msd4 / 1e6, "frac": bd4 / msd4 / 1e6 / HBM_PEAK_GBS}}
        log("Q4_K_M file mix: %.1f tok/s; Q4_K down 2560x9728 %.2f us (%.2f of peak)" % (mix["tok_s"], msd4 * 1e3, mix["q4k_down_2560x9728"]["frac"]))
        mdec.close()
        del mdec, mlayers
        torch.cuda.empty_cache()

    # ---- decode deep into a long chat: the same model with 8192 and 32768 cached positions (fp16 cache, 4.8 GB at 32 k) ----
    longctx = None
    if args.long_context:
        LMAX = 32768 + 256
        ldec2 = Decoder(cfg, layers, head, max_seq=LMAX, kv_fp16=True, use_graph=True)
        for i in range(cfg["n_layers"]):
            ldec2.k_cache[i].normal_()
            ldec2.v_cache[i].normal_()
        nh, nkv, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
        S2 = ops.flash_decode_num_splits(LMAX)
        q_ = torch.randn(nh * hd, device="cuda")
        k_ = torch.randn(nkv * hd, device="cuda")
        v_ = torch.randn(nkv * hd, device="cuda")
        w_ = torch.ones(hd, device="cuda")
        O_ = torch.empty(nh * hd, device="cuda")
        pO_ = torch.empty(S2 * nh * hd, device="cuda")
        pL_ = torch.empty(S2 * nh, device="cuda")
        pM_ = torch.empty(S2 * nh, device="cuda")
        rope_ = ops.rope_table(LMAX, hd, cfg["rope_base"]).cuda()
        longctx = {"max_seq": LMAX}
        for T in (2048, 8192, 32768):
            ldec2.set_past_len(T)
            ltok2 = 1
            for _ in range(4):
                ltok2 = ldec2.step(ltok2)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(32):
                ltok2 = ldec2.step(ltok2)
            torch.cuda.synchronize()
            ldt2 = (time.perf_counter() - t1) / 32
            past_ = torch.tensor([T + 20], dtype=torch.int64, device="cuda")
            msa = event_time_ms(lambda i: ops.attn_decode_fused(q_, k_, v_, w_, w_, ldec2.k_cache[i % 36], ldec2.v_cache[i % 36], O_, pO_, pL_, pM_,
                                                                rope_, nh, nkv, hd, past_, LMAX, hd ** -0.5, 1e-6), 72, torch)
            kvb = 2 * (T + 20) * nkv * hd * 2
            longctx["past_%d" % T] = {"tok_s": 1.0 / ldt2, "ms_per_token": ldt2 * 1e3, "attn_plus_merge_us": msa * 1e3,
                                      "kv_bytes_per_layer": kvb, "attn_GBs": kvb / msa / 1e6}
            log("past %d (cache of %d): %.1f tok/s, attention + merge %.1f us per layer (%.0f GB/s)" % (T, LMAX, 1.0 / ldt2, msa * 1e3, kvb / msa / 1e6))
        ldec2.close()
        del ldec2
        torch.cuda.empty_cache()

    # ---- CPU baseline on this host: bounded sample of the same workload ---------------------------
    cpu = None
    if args.cpu_tokens > 0:
        try:
            cpu = cpu_baseline(cfg, layers, head, kvs, args.cpu_tokens, child)
        except Exception as e:  # the baseline is reported, never required
            log("cpu baseline failed: %r" % (e,))
    out = {
        "metric": baseline["metric"], "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[3]: batch-1 greedy decode, Qwen3-4B-shaped Q4_K_M (36 layers, q/k/o/gate/up Q4_K, "
                               "v/down/lm_head Q6_K), fp16 KV prefilled 2048, %d new tokens" % args.steps,
                   "kv_cache": "fp16", "graph": "hipGraph per token", "host_sync": "per token"},
        "roofline": roof, "cpu_baseline": cpu, "gemv": gemv,
        "chained_tok_s": chained_tok_s, "chained_tokens_identical": bool(tokens_equal),
        "sampled_tok_s": sampled_tok_s, "sampled_chained_tok_s": sampled_chained_tok_s,
        "llama3_8b_shape": llama,
        "gemma3_4b_shape": gemma,
        "qwen25_7b_shape": q25,
        "q4km_file_type_mix": mix,
        "long_context": longctx,
        "a100_published_tok_s": 82.6, "x_a100_published": tok_s / 82.6,
        "token_hbm_frac": per_token_bytes / (dt / args.steps) / 1e9 / HBM_PEAK_GBS,
    }
    sys.stdout.flush()
    os.write(json_fd, (json.dumps(out) + "\n").encode())
    os.close(json_fd)


def cpu_measure(cfg, layers, head, kvs, n_tokens):
    """The reference's CPU path (oracle/_ref when built, else this repository's C port) on this host with however many
    threads its pool was created with: configs[0] / [1] / [2] as GB/s over the algorithmic bytes (median of 5 timed passes
    after a warm-up pass, weights beyond the host caches), configs[3] as tokens per second over n_tokens greedy tokens."""
    from oracle import pyoracle as po
    from prometorch_amd.testing import synth
    kind, model, cores = "port", None, None
    if po.have_ref():
        try:
            emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
            model = po.RefModel(cfg, layers, head, MAX_SEQ, emb)
            kind = "reference"
            cores = po.ref().ref_num_threads()
        except OSError as e:
            log("oracle/_ref not loadable (%r): timing the C port" % (e,))
    if model is None:
        model = po.OracleModel(cfg, layers, head, MAX_SEQ, kv_fp16=False)
        cores = po.lib().po_num_threads()
    gemv = po.ref_gemv if kind == "reference" else po.gemv
    H, I, V = cfg["hidden"], cfg["inter"], cfg["vocab"]
    nL = len(layers)

    def median5(fn):
        fn(0)
        ts = []
        for rep in range(5):
            t = time.perf_counter()
            fn(rep + 1)
            ts.append(time.perf_counter() - t)
        return sorted(ts)[2]

    out = {}
    xh = synth.make_x(synth.rng_for(SEED, 11), H)
    xi = synth.make_x(synth.rng_for(SEED, 12), I)
    xq = synth.make_x(synth.rng_for(SEED, 13), cfg["n_heads"] * cfg["head_dim"])
    # configs[0]: one Q4_K GEMV 9728 x 2560; a pass = 6 launches over 6 layers' gate matrices (84 MB), another 6 each pass
    n0 = 6
    b0 = layers[0]["gate"][1].size + 4 * H + 4 * I
    t0 = median5(lambda rep: [gemv(12, layers[(n0 * rep + i) % nL]["gate"][1], xh) for i in range(n0)]) / n0
    out["cfg0_q4k_gemv_9728x2560"] = {"us": t0 * 1e6, "GBs": b0 / t0 / 1e9}
    # configs[1]: Q6_K lm_head 151936 x 2560 + argmax (319 MB per pass)
    b1 = head["lm_head"].size + 4 * H + 4 * V
    t1 = median5(lambda rep: int(np.argmax(gemv(14, head["lm_head"], xh))))
    out["cfg1_q6k_lm_head_argmax"] = {"us": t1 * 1e6, "GBs": b1 / t1 / 1e9}
    # configs[2]: the seven GEMVs of one decoder layer in the Q4_K_M mix (64 MB), another layer each pass
    def layer_gemvs(rep):
        L = layers[rep % nL]
        for name, xx in (("q", xh), ("k", xh), ("v", xh), ("o", xq), ("gate", xh), ("up", xh), ("down", xi)):
            gemv(L[name][0], L[name][1], xx)
    b2 = sum(layers[0][n][1].size for n in ("q", "k", "v", "o", "gate", "up", "down"))
    t2 = median5(layer_gemvs)
    out["cfg2_layer_gemvs"] = {"us": t2 * 1e6, "GBs": b2 / t2 / 1e9}
    # configs[3]: greedy tokens of the whole model after one warm-up token
    for i, (k, v) in enumerate(kvs):
        model.set_kv(i, k, v)
    tok = model.step(1)
    t = time.perf_counter()
    for _ in range(n_tokens):
        tok = model.step(tok)
    dt = time.perf_counter() - t
    if hasattr(model, "close"):
        model.close()
    out["tok_s"] = n_tokens / dt
    out["tokens"] = n_tokens
    out["cores"] = int(cores)
    out["kind"] = kind
    log("cpu baseline (%s, %d threads): %.2f tok/s; cfg0 %.1f GB/s, cfg1 %.1f GB/s, cfg2 %.1f GB/s" %
        (kind, cores, out["tok_s"], out["cfg0_q4k_gemv_9728x2560"]["GBs"], out["cfg1_q6k_lm_head_argmax"]["GBs"],
         out["cfg2_layer_gemvs"]["GBs"]))
    return out


def cpu_child_main(n_tokens):
    """`bench.py --cpu-child N`: the CPU measurement alone, in a process of its own that never touches the GPU.  The parent
    starts it with PT_NUM_THREADS=1 (the reference sizes its thread pool once per process, c10/util/ThreadPool.h:96-109) before
    it initialises the GPU itself, and reads the JSON line this prints."""
    from prometorch_amd.testing import synth
    cfg = dict(synth.QWEN3_4B)
    layers = [synth.make_layer(SEED, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(SEED, cfg)
    kvs = [synth.make_kv_prefill(SEED, i, cfg, N_PREFILL) for i in range(cfg["n_layers"])]
    json_fd = os.dup(1)
    os.dup2(2, 1)
    res = cpu_measure(cfg, layers, head, kvs, n_tokens)
    os.write(json_fd, (json.dumps(res) + "\n").encode())


def cpu_baseline(cfg, layers, head, kvs, n_tokens, one_thread_child):
    """cpu_baseline of the JSON line: the T-thread measurement made here, the 1-thread one collected from the child."""
    full = cpu_measure(cfg, layers, head, kvs, n_tokens)
    one = None
    if one_thread_child is not None:
        try:
            stdout, _ = one_thread_child.communicate(timeout=600)
            one = json.loads(stdout.decode().strip().splitlines()[-1])
        except Exception as e:  # reported, never required
            log("1-thread cpu baseline failed: %r" % (e,))
    res = {"value": full["tok_s"], "unit": "tok/s", "cores": full["cores"], "kind": full["kind"],
           "sample": "%d greedy tokens of the same 36-layer model after 1 warm-up token, KV prefilled to %d (fp32 KV on the CPU); "
                     "configs[0..2]: median of 5 timed passes after a warm-up pass, GB/s over the algorithmic bytes" % (n_tokens, N_PREFILL),
           "cfg0_q4k_gemv_9728x2560": full["cfg0_q4k_gemv_9728x2560"], "cfg1_q6k_lm_head_argmax": full["cfg1_q6k_lm_head_argmax"],
           "cfg2_layer_gemvs": full["cfg2_layer_gemvs"]}
    if one is not None:
        res["one_thread"] = {"value": one["tok_s"], "unit": "tok/s", "cores": one["cores"], "tokens": one["tokens"],
                             "cfg0_q4k_gemv_9728x2560": one["cfg0_q4k_gemv_9728x2560"],
                             "cfg1_q6k_lm_head_argmax": one["cfg1_q6k_lm_head_argmax"], "cfg2_layer_gemvs": one["cfg2_layer_gemvs"]}
    return res


if __name__ == "__main__":
    main()
