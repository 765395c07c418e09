"""Writes the golden fixtures of this directory.  Run from the repo root: python tests/golden/make_golden.py

Expected values come from torch's CPU library routines (the arithmetic the reference delegates to):
  fbcache_*   eager bf16/fp16 ops of are_two_tensors_similar (src/para_attn/first_block_cache/utils.py:228-233)
  attention_* torch CPU SDPA (bf16 out + fp32 LSE), the oracle of src/para_attn/ops/__init__.py:160-179
  taylorseer_* eager ops evaluating the expressions of src/para_attn/first_block_cache/taylorseer.py:35,45
              and the cache-hit add of first_block_cache/utils.py:242
  merge_*     torch _SDPAMerger (torch/distributed/tensor/experimental/_context_parallel/_attention.py:138-223)
The reference holds no golden vectors of its own for these ops (tests/ops/test_ops.py:62 is a tautology).
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import inputs  # noqa: E402


def bf16_bits(t):
    return t.view(torch.int16).numpy().astype(np.uint16)


def fbcache():
    cases, arrays = [], {}
    specs = [
        ("hit_005", (1, 96, 64), 0.05, 0.12, torch.bfloat16),
        ("miss_020", (1, 96, 64), 0.20, 0.12, torch.bfloat16),
        ("edge_0119", (1, 700, 64), 0.1190, 0.12, torch.bfloat16),
        ("edge_0120", (1, 700, 64), 0.1200, 0.12, torch.bfloat16),
        ("edge_0121", (1, 700, 64), 0.1210, 0.12, torch.bfloat16),
        ("hunyuan_006", (2, 48, 128), 0.07, 0.06, torch.bfloat16),
        ("f16_hit", (1, 96, 64), 0.05, 0.08, torch.float16),
        ("f16_miss", (1, 96, 64), 0.15, 0.08, torch.float16),
        ("odd_tail", (1, 7, 13), 0.1, 0.12, torch.bfloat16),
    ]
    for i, (name, shape, noise, thr, dtype) in enumerate(specs):
        prev, cur = inputs.fbcache_pair(shape, seed=100 + i, noise=noise, dtype=dtype)
        mean_diff = (prev - cur).abs().mean()
        mean_t1 = prev.abs().mean()
        ratio = (mean_diff / mean_t1).item()
        if dtype == torch.bfloat16:
            arrays[name + "_prev"], arrays[name + "_cur"] = bf16_bits(prev), bf16_bits(cur)
        else:
            arrays[name + "_prev"], arrays[name + "_cur"] = prev.numpy(), cur.numpy()
        cases.append({
            "name": name, "dtype": "bf16" if dtype == torch.bfloat16 else "f16", "threshold": thr,
            "ratio": ratio, "mean_diff": mean_diff.item(), "mean_t1": mean_t1.item(), "similar": ratio < thr,
        })
    np.savez_compressed(os.path.join(HERE, "fbcache_inputs.npz"), **arrays)
    with open(os.path.join(HERE, "fbcache_cases.json"), "w") as f:
        json.dump(cases, f, indent=1)


def attention():
    arrays = {}
    for name, (B, H, Sq, Skv, D) in {"a": (1, 2, 34, 120, 128), "b": (2, 1, 129, 17, 64)}.items():
        q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=7)
        out, lse = torch.ops.aten._scaled_dot_product_flash_attention_for_cpu(q, k, v)
        for n, t in (("q", q), ("k", k), ("v", v), ("out", out)):
            arrays[f"{name}_{n}"] = bf16_bits(t)
        arrays[f"{name}_lse"] = lse.numpy()
    np.savez_compressed(os.path.join(HERE, "attention_cases.npz"), **arrays)


def merge():
    from torch.distributed.tensor.experimental._context_parallel._attention import _SDPAMerger

    g = torch.Generator().manual_seed(11)
    outs = [torch.randn(1, 2, 19, 32, generator=g).bfloat16() for _ in range(4)]
    lses = [torch.randn(1, 2, 19, generator=g) * 5 for _ in range(4)]
    m = _SDPAMerger(True, 2)
    arrays = {}
    for i, (o, l) in enumerate(zip(outs, lses)):
        m.step(o, l, False)
        arrays[f"out{i}"], arrays[f"lse{i}"] = bf16_bits(o), l.numpy()
        arrays[f"acc_out{i}"], arrays[f"acc_lse{i}"] = m._out.float().numpy().copy(), m._lse.squeeze(-1).numpy().copy()
    ro, rl = m.results()
    arrays["result_out"], arrays["result_lse"] = bf16_bits(ro), rl.numpy()
    np.savez_compressed(os.path.join(HERE, "merge_cases.npz"), **arrays)


def taylorseer():
    import math

    arrays, cases = {}, []
    g = torch.Generator().manual_seed(23)
    specs = [  # name, dtype, shape, orders of difference / stored orders, window, elapsed
        ("bf16_w1", torch.bfloat16, (1, 37, 23), 2, 1, 1),
        ("bf16_w3", torch.bfloat16, (1, 37, 23), 2, 3, 2),
        ("bf16_o4", torch.bfloat16, (2, 16, 40), 4, 5, 3),
        ("f16_w3", torch.float16, (1, 37, 23), 2, 3, 2),
        ("f32_w3", torch.float32, (1, 9, 7), 3, 3, 4),
    ]
    for name, dtype, shape, n, window, elapsed in specs:
        y = (torch.randn(shape, generator=g) * 2).to(dtype)
        prev = [(torch.randn(shape, generator=g) * (2.0 / (i + 1))).to(dtype) for i in range(n)]
        hidden = torch.randn(shape, generator=g).to(dtype)
        # approximate_derivative (taylorseer.py:33-35)
        cur = [y]
        for i in range(n):
            cur.append((cur[i] - prev[i]) / window)
        # approximate_value (taylorseer.py:42-47) over the orders just built
        output = 0
        for i, derivative in enumerate(cur):
            output += (1 / math.factorial(i)) * derivative * (elapsed**i)
        applied = output + hidden  # utils.py:242
        enc = bf16_bits if dtype == torch.bfloat16 else (lambda t: t.numpy())
        arrays[name + "_y"], arrays[name + "_hidden"] = enc(y), enc(hidden)
        for i in range(n):
            arrays[f"{name}_prev{i}"], arrays[f"{name}_cur{i + 1}"] = enc(prev[i]), enc(cur[i + 1])
        arrays[name + "_value"], arrays[name + "_applied"] = enc(output), enc(applied)
        cases.append({"name": name, "dtype": {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[dtype],
                      "n": n, "window": window, "elapsed": elapsed})
    arrays["cases"] = np.array(json.dumps(cases))
    np.savez_compressed(os.path.join(HERE, "taylorseer_cases.npz"), **arrays)


if __name__ == "__main__":
    fbcache()
    taylorseer()
    attention()
    merge()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith((".npz", ".json"))))
