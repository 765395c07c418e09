"""Headline benchmark: attention_forward_with_lse at the 119k-token HunyuanVideo head-share shape
(B=1, 3 of 24 heads, S=119056, D=128, bf16, q/k RMS-normalised), one MI355X.

Prints ONE JSON line.  ``value`` is attention TFLOP/s (4*B*H*Sq*Skv*D flop per call) with inputs
resident in HBM; ``roofline`` prices the attention kernel against the bf16 dense MFMA peak;
``cpu_baseline`` is torch's CPU SDPA (the library routine the reference's SDPA path is checked
against) on a bounded sample of the same workload; ``extras`` holds the bandwidth-bound kernels
(ring merge step, FBCache reduction) against the HBM peak.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E


def _time_calls(fn, steps, warmup):
    """Average milliseconds per call over ``steps`` calls, HIP events on the current stream."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (use --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    import paraattention_amd  # noqa: F401
    from paraattention_amd import _lib
    from oracle import inputs

    _lib.load()  # no fallback: a missing library is an error
    dev = torch.device("cuda:0")
    B, H, S, D = 1, 3, 119056, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=0, rms_norm_qk=True)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    flops = 4.0 * B * H * S * S * D

    op = torch.ops.para_attn.attention_forward_with_lse
    ms_evt, ms_wall = _time_calls(lambda: op(qd, kd, vd), args.steps, args.warmup)
    tflops = flops / (ms_wall * 1e-3) / 1e12
    kern_tflops = flops / (ms_evt * 1e-3) / 1e12

    result = {
        "metric": "attn TFLOP/s & % bf16 MFMA peak at 119k-token HunyuanVideo shape; ms/call",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_wall, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "HunyuanVideo 720p single-rank Ulysses head share: attention_forward_with_lse "
                        "B=1 H=3 Sq=Skv=119056 D=128 bf16, q/k RMS-normalised, non-causal, out + fp32 LSE",
            "flop_per_call": flops,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "attn_fwd_kernel<BF16,128,dense>",
            "achieved": round(kern_tflops, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(kern_tflops / PEAK_BF16_TFLOPS, 4),
            "ms_per_launch": round(ms_evt, 4),
            "traffic": None,
        },
    }

    if not args.no_extras:
        extras = {}
        # ring merge step at the ring-sweep shape: fp32 accumulator updated in place by a bf16 partial
        Bm, Hm, Sm = 1, 24, 14882
        g = torch.Generator().manual_seed(1)
        acc = torch.randn(Bm, Hm, Sm, D, generator=g).to(dev)
        acc_l = torch.randn(Bm, Hm, Sm, generator=g).to(dev)
        blk = torch.randn(Bm, Hm, Sm, D, generator=g).bfloat16().to(dev)
        blk_l = torch.randn(Bm, Hm, Sm, generator=g).to(dev)
        mop = torch.ops.para_attn.merge_attention_lse_
        ms, _ = _time_calls(lambda: mop(acc, acc_l, blk, blk_l), 20, 3)
        mbytes = Bm * Hm * Sm * D * 10 + Bm * Hm * Sm * 12
        extras["merge_lse"] = {
            "workload": "ring merge step, acc fp32 [1,24,14882,128] in place, partial bf16",
            "bound": "hbm", "bytes_per_launch": mbytes, "ms_per_launch": round(ms, 4),
            "achieved": round(mbytes / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(mbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        }
        del acc, blk
        # FBCache reduction at the Wan first-block residual shape
        prev, cur = inputs.fbcache_pair((1, 32760, 5120), seed=1234)
        pd, cd = prev.to(dev), cur.to(dev)
        fop = torch.ops.para_attn.fbcache_residual_diff
        ms, _ = _time_calls(lambda: fop(pd, cd), 20, 3)
        fbytes = 4 * prev.numel()
        extras["fbcache_residual_diff"] = {
            "workload": "bf16 [1,32760,5120] residual pair", "ratio": fop(pd, cd).item(),
            "bound": "hbm", "bytes_per_launch": fbytes, "ms_per_launch": round(ms, 4),
            "achieved": round(fbytes / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(fbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        }
        del pd, cd
        result["extras"] = extras

    if not args.no_cpu_baseline:
        from oracle import attention as oattn

        rows = 16384  # bounded sample: one head, the first 16384 query rows against all 119056 keys
        cores = torch.get_num_threads()
        qs, ks, vs = q[:, :1, :rows].contiguous(), k[:, :1].contiguous(), v[:, :1].contiguous()
        oattn.sdpa_lse_torch_cpu(qs[:, :, :512], ks, vs)  # warm the thread pool
        t0 = time.perf_counter()
        oattn.sdpa_lse_torch_cpu(qs, ks, vs)
        dt = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": round(4.0 * rows * S * D / dt / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": cores,
            "kind": "port",
            "sample": f"torch CPU SDPA (bf16 out + fp32 LSE), 1 head, first {rows} of {S} query rows x all {S} keys, {dt:.2f} s",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
