#!/usr/bin/env python3
"""Decode-attention benchmark of the KV-cache hot path on one MI355X.

Workload (BASELINE.json configs[2], the configuration the metric is quoted on):
QuantizedKVCache, 4-bit, group 64, Llama-3-8B attention shape (32 query heads,
8 KV heads, head_dim 128), batch 32, fp16, context prefilled to 32768 tokens.
One step = one pass of the hot path over one batch: quantize-on-append of one new
token per sequence, then fused dequantize + scaled-dot-product attention over the
whole cached context (one layer).  Inputs are synthetic (K/V ~ N(0,1) times a
per-channel scale drawn log-uniform in [0.1, 10]; Q ~ N(0,1), seed 0) and are
resident in HBM before the timed region starts.

Prints one JSON line: decode tokens/s (= batch / step time), plus
  roofline     achieved HBM GB/s of the dominant kernel (split-sequence decode
               attention): algorithmic bytes per launch B*Hkv*T*144 divided by its
               mean duration, measured with HIP events on the launch stream
  cpu_baseline the CPU restatement of the reference's unfused op sequence
               (oracle/kv_oracle.c), timed here on the host cores on a bounded
               sample of the same workload, and used to check the GPU output.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "mlx-swift-lm_amd"))

B, HQ, HKV, D, BITS, GS, CTX = 32, 32, 8, 128, 4, 64, 32768
HBM_PEAK_GBS = 8000.0
# HBM bytes moved per launch of the decode kernel divided by its algorithmic bytes, from two
# rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by what the same counters read for a
# plain 1 GiB copy; summary in profiles/decode_kernel_q4_d128_cfg3.md
MEASURED_TRAFFIC_RATIO = 1.0033
ROW_BYTES = 144  # per cached token and kv head: K and V codes 2*64 B + 2*2 groups*(scale+bias)*2 B


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--context", type=int, default=CTX)
    ap.add_argument("--batch", type=int, default=B)
    ap.add_argument("--cpu-steps", type=int, default=2, help="decode steps timed on the CPU baseline (0 = skip)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy 4 times (reference point for rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--traffic-kib", type=float, default=None,
                    help="HBM KiB per launch of the decode kernel from rocprofv3 --pmc runs (else null)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus above 1 is not supported "
              "(the path shards over batch / KV heads without exchange, see DESIGN.md)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import kvhip
    from kvhip import _lib as L

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; libkvhip has no CPU path", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    nb, ctx = args.batch, args.context
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    ch = (10.0 ** (torch.rand(D, generator=g, device=dev) * 2 - 1)).to(torch.float32)

    cache = kvhip.QuantizedKVCache(GS, BITS)
    total = ctx + args.warmup + args.steps + 8
    cache.reserve(nb, HKV, D, D, torch.float16, total)
    chunk = 2048
    for t0 in range(0, ctx, chunk):
        n = min(chunk, ctx - t0)
        k = (torch.randn(nb, HKV, n, D, generator=g, device=dev) * ch).to(torch.float16)
        v = (torch.randn(nb, HKV, n, D, generator=g, device=dev) * ch).to(torch.float16)
        cache.update_quantized(k, v, fetch=False)
    del k, v
    nsteps = args.warmup + args.steps
    qs = torch.randn(nsteps, nb, HQ, 1, D, generator=g, device=dev).to(torch.float16)
    ks = (torch.randn(nsteps, nb, HKV, 1, D, generator=g, device=dev) * ch).to(torch.float16)
    vs = (torch.randn(nsteps, nb, HKV, 1, D, generator=g, device=dev) * ch).to(torch.float16)
    scale = 1.0 / D ** 0.5
    torch.cuda.synchronize()

    lib = kvhip.load()
    if args.calibrate_copy:
        src = torch.full((1 << 30,), 7, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for i in range(args.warmup):
        out = cache.update_attend(qs[i], ks[i], vs[i], scale)
    torch.cuda.synchronize()
    lib.kvhip_profile_enable(1)
    t_first = cache.offset + 1
    t0 = time.perf_counter()
    for i in range(args.warmup, nsteps):
        out = cache.update_attend(qs[i], ks[i], vs[i], scale)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    lib.kvhip_profile_enable(0)
    launches, kms = C.c_int32(), C.c_double()
    L.check(lib.kvhip_profile_read(C.byref(launches), C.byref(kms)))
    t_last = cache.offset
    elapsed = t1 - t0
    ms_per_step = 1e3 * elapsed / args.steps
    tok_s = nb * args.steps / elapsed

    mean_t = 0.5 * (t_first + t_last)
    alg_bytes = nb * HKV * mean_t * ROW_BYTES
    roofline = None
    if launches.value > 0:
        kernel_ms = kms.value / launches.value
        achieved = alg_bytes / (kernel_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": "decode_kernel<4,128,64,f16>", "achieved": round(achieved, 1),
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                    "kernel_ms": round(kernel_ms, 5), "algorithmic_bytes": int(alg_bytes),
                    "traffic": int(args.traffic_kib * 1024) if args.traffic_kib is not None
                    else (int(alg_bytes * MEASURED_TRAFFIC_RATIO) if (nb, ctx) == (B, CTX) else None)}

    # ---- CPU baseline + full-size parity sample ------------------------------------
    cpu = None
    parity = None
    if args.cpu_steps > 0:
        from oracle import c_oracle as CO
        from oracle import kv_oracle as O
        st = [a.cpu().numpy() for a in cache.state]
        kq = (st[0].view(np.uint32), st[1].astype(np.float32), st[2].astype(np.float32))
        vq = (st[3].view(np.uint32), st[4].astype(np.float32), st[5].astype(np.float32))
        q_last = qs[nsteps - 1].float().cpu().numpy()
        gpu_last = out.float().cpu().numpy()
        threads = CO.num_threads()
        tc0 = time.perf_counter()
        for _ in range(args.cpu_steps):
            ref = CO.qsdpa(q_last, kq, vq, scale, None, GS, BITS, "float16")
        tc1 = time.perf_counter()
        cpu_tok_s = nb * args.cpu_steps / (tc1 - tc0)
        cpu = {"value": round(cpu_tok_s, 3), "unit": "tokens/s", "cores": threads, "kind": "port",
               "sample": f"{args.cpu_steps} decode attention steps at B={nb}, T={t_last} "
                         f"(oracle/kv_oracle.c kvo_qsdpa, OpenMP; restated reference CPU path, not MLX)"}
        d = np.abs(gpu_last.astype(np.float64) - ref.astype(np.float64))
        parity = {"max_abs": float(d.max()), "mean_abs": float(d.mean()), "vs": "oracle at full size, last step"}

    line = {
        "metric": "KV-attn decode tok/s + HBM GB/s (% of peak), Llama-3-8B shape 4-bit KV 32k",
        "value": round(tok_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (4-bit affine codes, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "configs[2]: QuantizedKVCache 4-bit g64, 32q/8kv heads, head_dim 128, "
                               f"batch {nb}, context {ctx}+, quantize-on-append + fused dequant-SDPA, one layer",
                   "batch": nb, "context_first": int(t_first), "context_last": int(t_last)},
        "roofline": roofline, "cpu_baseline": cpu, "parity": parity,
        "hbm_gbs_whole_step": round(alg_bytes / (ms_per_step * 1e-3) / 1e9, 1),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
