"""Headline benchmark: attention_forward_with_lse at the 119k-token HunyuanVideo head-share shape
(B=1, 3 of 24 heads, S=119056, D=128, bf16, q/k RMS-normalised), one MI355X.

Prints ONE JSON line.  ``value`` is attention TFLOP/s (4*B*H*Sq*Skv*D flop per call) with inputs
resident in HBM (a call = everything the op launches: the score bound's two small kernels, both
variants of the attention kernel, one of which returns at once, and the merge of the partial results); ``roofline`` prices the call against the bf16
dense MFMA peak; ``cpu_baseline`` is torch's CPU SDPA (the library routine the reference's SDPA path
is checked against) on a bounded sample of the same workload; ``extras`` holds the other
configurations of the baseline (FLUX joint attention, the ring sweep, the Wan self- and
cross-attention legs, block-sparse attention) against the MFMA peak and the bandwidth-bound kernels
(ring merge step, FBCache reduction, TaylorSeer) against the HBM peak.

Every timed loop takes per-call HIP events on the launch stream and reports mean, median and
minimum.  What is reported is the steady state of a loop that keeps the GPU busy, which is what a diffusion
model's step is: after an idle gap the chip needs some tenths of a second of work to settle (measured: the
headline call takes 17.61 ms after 3 warm-up calls, 17.50 after 10, 17.40 after 30; FLUX joint attention 0.298 ms
after 5, 0.258 after 50, 0.255 after 200; the bandwidth-bound kernels move the other way, 2-3 % faster right after
the gap), so the defaults warm every loop up for that long (30 calls of the headline, 60-100 of the short kernels); the bandwidth-bound kernels rotate over several buffer sets so that the 256 MB
memory-side cache cannot hold a working set from one call to the next; a sample of rows of the last
timed output of every attention shape is compared with torch's CPU SDPA (``checked``).

``--only {attn,merge,fbcache,taylorseer,sparse,ring,flux,wan,shapes,copy,yardsticks,wave_rows}`` runs a single loop (what
the rocprofv3 summaries under profiles/ were taken with).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# Traffic at the L2's memory side per launch in bytes: FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 from two
# rocprofv3 --pmc runs of `bench.py --only <kernel>` (scale factors from a 1 GiB copy).  These counters cannot be
# read from inside this process; the figures are those of the summary named in TRAFFIC_SOURCE, not of this run.
TRAFFIC = {"attn": 1.005e10, "merge": 4.773e8, "fbcache": 6.710e8, "taylorseer": 1.677e9, "sparse": 8.940e9,
           "flux": 3.039e8, "ring_sweep": 1.234e10, "ring_sweep_per_block": 1.509e10, "wan_self": 3.797e9, "wan_cross": 7.013e8,
           "causal": 5.153e9, "text_mask": 1.005e10, "head_dim_64": 2.438e9}
TRAFFIC_SOURCE = "profiles/kernels_bench_workloads.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of the same command)"


def _time_calls(fn, steps, warmup):
    """Times ``steps`` calls of ``fn(i)`` after ``warmup`` untimed ones.

    Every call sits between two HIP events of its own on the launch stream (torch's current stream, the one
    the ops launch on); the loop as a whole is bracketed by synchronisations and the host clock.  Returns a
    dict: ``mean`` = first event to last event / steps, ``median`` and ``min`` over the per-call event times,
    ``wall`` = host clock / steps, all in ms.
    """
    import torch

    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        fn(warmup + i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per_call = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
    return {"mean": marks[0].elapsed_time(marks[steps]) / steps, "median": statistics.median(per_call),
            "min": min(per_call), "wall": wall_ms / steps}


def _ms_fields(t):
    return {"ms_per_launch": round(t["mean"], 4), "ms_median": round(t["median"], 4), "ms_min": round(t["min"], 4)}


def _hbm(name, workload, nbytes, t, sets):
    """Entry of a bandwidth-bound kernel: algorithmic bytes over the median launch time."""
    gbs = nbytes / (t["median"] * 1e-3) / 1e9
    return {
        "workload": workload, "bound": "hbm", "bytes_per_launch": nbytes, **_ms_fields(t),
        "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
        "buffer_sets_rotated": sets, "traffic": TRAFFIC.get(name), "traffic_source": TRAFFIC_SOURCE,
    }


def _mfma(workload, flops, t, **more):
    """Entry of an attention shape: algorithmic flops over the median time of one call."""
    tf = flops / (t["median"] * 1e-3) / 1e12
    return {"workload": workload, "bound": "mfma", "flop": flops, **_ms_fields(t), "achieved": round(tf, 2),
            "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), **more}


def _check_rows(out, lse, q, k, v, heads, rows, what, causal=False):
    """Compares sampled query rows of a timed call's output with torch's CPU SDPA on the same bits (the routine
    the oracle is pinned to); raises if they differ by more than the parity tolerance, else returns True.
    ``causal``: the sampled rows see keys 0..row only (is_causal of the full problem, as a mask for the sample)."""
    import torch

    from oracle import attention as oattn

    rows = torch.as_tensor(rows)
    keep = (torch.arange(k.shape[2])[None, :] <= rows[:, None])[None, None] if causal else None
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, heads][:, :, rows].contiguous(), k[:, heads].contiguous(), v[:, heads].contiguous(),
                                                attn_mask=keep)
    got = out[:, heads][:, :, rows.to(out.device)].float().cpu()
    err = (got - ref_out.float()).abs()
    if not bool((err <= 2e-2 + 2e-2 * ref_out.float().abs()).all()):
        raise AssertionError(f"{what}: timed output differs from the CPU oracle (max err {err.max().item():.4g})")
    if lse is not None:
        lerr = (lse[:, heads][:, :, rows.to(lse.device)].cpu() - ref_lse).abs().max().item()
        if lerr > 1e-3:
            raise AssertionError(f"{what}: timed LSE differs from the CPU oracle (max err {lerr:.4g})")
    return True


def _sample_rows(S, n=48, seed=1):
    import torch

    return torch.cat([torch.arange(0, 8), torch.arange(S - 8, S),
                      torch.randint(0, S, (n - 16,), generator=torch.Generator().manual_seed(seed))])


# ---------------------------------------------------------------------------------------------------------
# attention shapes (MFMA bound)
# ---------------------------------------------------------------------------------------------------------
def bench_attn(dev, steps, warmup):
    """The headline: the 119k-token HunyuanVideo head share."""
    import torch

    from oracle import inputs

    B, H, S, D = 1, 3, 119056, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=0, rms_norm_qk=True)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    op = torch.ops.para_attn.attention_forward_with_lse
    last = {}

    def call(i):
        last["out"], last["lse"] = op(qd, kd, vd)

    t = _time_calls(call, steps, warmup)
    checked = _check_rows(last["out"], last["lse"], q, k, v, [0, 1, 2], _sample_rows(S), "headline")
    return (q, k, v), 4.0 * B * H * S * S * D, t, checked


def _dense_case(dev, name, B, H, Sq, Skv, D, steps, warmup, seed=3, check_heads=(0,), traffic=None, causal=False, sets=1,
                masked_keys=0, shards=1):
    """One dense shape: timed, then sampled rows of the last timed output checked against torch's CPU SDPA.
    ``sets`` > 1: the calls rotate over that many copies of q, k, v at different addresses, so that a working set
    smaller than the 256 MB memory-side cache is not served from it call after call (in a model every call brings
    other tensors).  ``masked_keys`` > 0: the call passes a boolean key mask [1,1,1,Skv] that drops that many keys
    (a padded text prompt of 256 tokens): at the end, or with ``shards`` > 1 where the padding lies when that many
    ranks' [latent, text] shards have been gathered along the sequence, which is the mask the reference's
    sequence-parallel HunyuanVideo adapter builds (context_parallel/diffusers_adapters/hunyuan_video.py:86-100);
    flops and the check are those of the kept keys."""
    import torch

    from oracle import inputs

    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=seed)
    bufs = [(q.to(dev), k.to(dev), v.to(dev)) for _ in range(sets)]
    op = torch.ops.para_attn.attention_forward_with_lse
    last = {}
    kept = Skv - masked_keys
    keep = None
    if masked_keys:
        pos = torch.arange(Skv)
        shard, text = Skv // shards, 256 // shards
        text_index = (pos // shard) * text + (pos % shard - (shard - text))  # position in the prompt, for text tokens
        keep = (pos % shard < shard - text) | (text_index < 256 - masked_keys) | (pos >= shards * shard)
        assert int(keep.sum()) == kept
    mask = keep[None, None, None, :].to(dev) if masked_keys else None

    def call(i):
        qd, kd, vd = bufs[i % sets]
        last["out"], last["lse"] = op(qd, kd, vd, mask, is_causal=causal)

    t = _time_calls(call, steps, warmup)
    heads = sorted(set(list(check_heads) + [H - 1]))
    k_kept, v_kept = (k, v) if keep is None else (k[:, :, keep], v[:, :, keep])
    checked = _check_rows(last["out"], last["lse"], q, k_kept, v_kept, heads, _sample_rows(Sq), name, causal=causal)
    flops = 4.0 * B * H * Sq * kept * D * (0.5 if causal else 1.0)  # causal: the kept half (Sq == Skv)
    nbytes = 2.0 * B * H * D * (2 * Sq + 2 * Skv) + 4.0 * B * H * Sq
    gbs = nbytes / (t["median"] * 1e-3) / 1e9
    more = {"traffic": TRAFFIC[traffic], "traffic_source": TRAFFIC_SOURCE} if traffic else {}
    if sets > 1:
        more["buffer_sets"] = sets
    what = "attention_forward_with_lse" + (" is_causal" if causal else "")
    if masked_keys:
        what += f" with a key mask that drops {masked_keys} keys" + (" at the end" if shards == 1 else f" in the text parts of {shards} gathered shards")
    return _mfma(f"{name}: {what} q [{B},{H},{Sq},{D}] k,v [{B},{H},{Skv},{D}] bf16", flops, t,
                 bytes=nbytes, gbs=round(gbs, 1), frac_hbm=round(gbs / PEAK_HBM_GBS, 4), checked=checked, **more)


def bench_flux(dev, steps=50, warmup=100):
    """FLUX-dev joint attention.  q, k, v and the output are 113 MB together, less than the memory-side cache: four
    sets of inputs are rotated."""
    return _dense_case(dev, "FLUX joint attention", 1, 24, 4608, 4608, 128, steps, warmup, seed=0, traffic="flux", sets=4)


def bench_wan(dev, steps=10, warmup=10):
    """Both attention legs of a Wan 2.1 block.  Cross-attention to 512 keys sits near the ridge: both bounds."""
    return {
        "wan_self_attention": _dense_case(dev, "Wan 2.1 self-attention", 1, 40, 32760, 32760, 128, steps, warmup, seed=4, check_heads=(0, 17), traffic="wan_self"),
        "wan_cross_attention": _dense_case(dev, "Wan 2.1 cross-attention to 512 text keys", 1, 40, 32760, 512, 128, 4 * steps, 10 * warmup, seed=2, check_heads=(0, 17), traffic="wan_cross"),
    }


def bench_ring(dev, steps=6, warmup=3):
    """One rank's ring pass: a Q block of 14882 tokens x 24 heads against 8 KV blocks of 14882 keys; checked against
    one SDPA over all 119056 keys.  Two ways: all blocks in one launch (the softmax state carried across the blocks
    in registers: what a sweep over resident blocks is), and one launch per block with the fp32 running pair folded
    inside the attention kernel (what a rank of a real ring does as blocks arrive)."""
    import torch

    import paraattention_amd

    B, H, S, D, nblk = 1, 24, 14882, 128, 8
    g = torch.Generator().manual_seed(2)
    q = torch.randn(B, H, S, D, generator=g).bfloat16()
    kb_cpu = [torch.randn(B, H, S, D, generator=g).bfloat16() for _ in range(nblk)]
    vb_cpu = [torch.randn(B, H, S, D, generator=g).bfloat16() for _ in range(nblk)]
    qd, kb, vb = q.to(dev), [t.to(dev) for t in kb_cpu], [t.to(dev) for t in vb_cpu]
    heads = [0, H - 1]
    k_all = torch.cat([kk[:, heads] for kk in kb_cpu], dim=2)
    v_all = torch.cat([vv[:, heads] for vv in vb_cpu], dim=2)
    flops = 4.0 * B * H * S * S * nblk * D
    out = {}
    for key, fused, launches, how in (
        ("ring_sweep", "sweep", 1, "one launch over all blocks, softmax state carried in registers"),
        ("ring_sweep_per_block", True, nblk, "one launch per block, fp32 running pair folded inside the attention kernel"),
    ):
        last = {}

        def call(i):
            last["out"], last["lse"] = paraattention_amd.ring_sweep(qd, kb, vb, fused=fused)

        t = _time_calls(call, steps, warmup)
        checked = _check_rows(last["out"][:, heads], last["lse"][:, heads], q[:, heads], k_all, v_all, [0, 1], _sample_rows(S), key)
        out[key] = _mfma(f"ring sweep: Q block [1,24,14882,128] bf16 against 8 KV blocks of 14882 keys, {how}", flops, t,
                         launches_per_sweep=launches, checked=checked, traffic=TRAFFIC[key], traffic_source=TRAFFIC_SOURCE)
    return out


def bench_shapes(dev, steps=10, warmup=5):
    """Further dense shapes: the headline shape with is_causal (flops of the kept half), the headline shape with the
    key mask of a padded text prompt (as a prefix, and as it lies in the sequence gathered from 8 ranks), and a
    head_dim 64 shape."""
    return {
        "headline_shape_causal": _dense_case(dev, "headline shape", 1, 3, 119056, 119056, 128, steps, warmup, seed=5,
                                             check_heads=(0, 1), causal=True, traffic="causal"),
        "headline_shape_text_mask": _dense_case(dev, "headline shape", 1, 3, 119056, 119056, 128, steps, warmup, seed=7,
                                                check_heads=(0, 1), masked_keys=167, traffic="text_mask"),
        "headline_shape_text_mask_8_shards": _dense_case(dev, "headline shape", 1, 3, 119056, 119056, 128, steps, warmup, seed=8,
                                                         check_heads=(0, 1), masked_keys=167, shards=8),
        "head_dim_64": _dense_case(dev, "head_dim 64 (CogVideoX-like)", 1, 48, 17776, 17776, 64, steps, warmup, seed=6,
                                   check_heads=(0, 23), traffic="head_dim_64"),
    }


def bench_wave_rows(dev, steps=12, warmup=20):
    """The resident-workgroup kernel as 8 wavefronts of 32 query rows (what ships) against 4 wavefronts of 64 (knob
    "wave_rows"), alternating twice in one process on the same tensors: median ms and fraction of the MFMA peak per
    setting and shape.  The two forms give the same bits, which is checked."""
    import statistics as st

    import torch

    from oracle import inputs
    from paraattention_amd import _lib

    op = torch.ops.para_attn.attention_forward_with_lse
    out = {}
    shapes = [("headline", 1, 3, 119056, 119056, True), ("wan_self", 1, 40, 32760, 32760, False),
              ("ring_block", 1, 24, 14882, 14882, False), ("flux", 1, 24, 4608, 4608, False), ("wan_cross", 1, 40, 32760, 512, False)]
    try:
        for name, B, H, Sq, Skv, rms in shapes:
            q, k, v = (t.to(dev) for t in inputs.qkv(B, H, Sq, Skv, 128, seed=0, rms_norm_qk=rms))
            flops = 4.0 * B * H * Sq * Skv * 128
            long = flops > 1e13
            ref, rows = None, {32: [], 64: []}
            for _ in range(2):
                for wr in (32, 64):
                    _lib.set_tuning("wave_rows", wr)
                    t = _time_calls(lambda i: op(q, k, v), steps if long else 4 * steps, warmup if long else 5 * warmup)
                    rows[wr].append(t["median"])
                    o, l = op(q, k, v)
                    if ref is None:
                        ref = (o, l)
                    elif not (torch.equal(o, ref[0]) and torch.equal(l, ref[1])):
                        raise AssertionError(f"{name}: the two wavefront forms differ")
            out[name] = {f"rows_{wr}": {"ms_median": round(st.median(ms), 4), "frac": round(flops / (st.median(ms) * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}
                         for wr, ms in rows.items()}
            del q, k, v
    finally:
        _lib.set_tuning("wave_rows", 0)
    return out


def bench_sparse(dev, steps=10, warmup=10):
    import torch

    from oracle import inputs

    B, H, S, D, nb = 1, 24, 32768, 128, 256
    q, k, v = inputs.qkv(B, H, S, S, D, seed=0)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    mask, density = inputs.block_mask(H, nb, nb, seed=0)
    md = mask.to(dev)
    op = torch.ops.para_attn.attention_forward_block_sparse
    last = {}

    def call(i):
        last["out"], last["lse"] = op(qd, kd, vd, md)

    t = _time_calls(call, steps, warmup)
    # check: two query blocks of two heads against dense SDPA over their kept key blocks, gathered
    checked = True
    blk = S // nb
    for h, qb in ((0, 0), (H - 1, nb // 2 + 3)):
        kept = mask[h, qb].nonzero().flatten()
        cols = (kept[:, None] * blk + torch.arange(blk)[None, :]).flatten()
        rows = torch.arange(qb * blk, (qb + 1) * blk)
        checked &= _check_rows(last["out"][:, h:h + 1], last["lse"][:, h:h + 1], q[:, h:h + 1], k[:, h:h + 1][:, :, cols],
                               v[:, h:h + 1][:, :, cols], [0], rows, "block-sparse")
    flops = 4.0 * B * H * S * S * D * density
    r = _mfma("block-sparse attention B1 H24 S32768 D128 bf16, 128x128 tiles, per-(head,q-block) mask", flops, t,
              density=round(density, 4), checked=checked, traffic=TRAFFIC["sparse"], traffic_source=TRAFFIC_SOURCE)
    # second bound: the tile transport.  Every kept tile is copied into LDS once per query block
    # (2 x 32 KB per 128x128 tile); what of that misses the L2s is `traffic`, priced against the HBM peak.
    copied = 2.0 * B * H * nb * nb * density * blk * D * 2
    gbs = TRAFFIC["sparse"] / (t["median"] * 1e-3) / 1e9
    r["transport"] = {"bound": "hbm", "tile_bytes_copied_to_lds": copied, "l2_miss_bytes": TRAFFIC["sparse"],
                      "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}
    return r


# ---------------------------------------------------------------------------------------------------------
# bandwidth-bound kernels: each loop rotates over SETS buffer sets (working sets of 0.27 - 1.7 GB each)
# ---------------------------------------------------------------------------------------------------------
SETS = 3


def bench_merge(dev, steps=30, warmup=60):
    import torch

    # ring merge step at the ring-sweep shape: fp32 accumulator updated in place by a bf16 partial
    B, H, S, D = 1, 24, 14882, 128
    g = torch.Generator(device=dev).manual_seed(1)  # drawn on the device: parity of this kernel is the tests' business
    sets = []
    for _ in range(SETS):
        sets.append((torch.randn(B, H, S, D, generator=g, device=dev), torch.randn(B, H, S, generator=g, device=dev),
                     torch.randn(B, H, S, D, generator=g, device=dev).bfloat16(), torch.randn(B, H, S, generator=g, device=dev)))
    op = torch.ops.para_attn.merge_attention_lse_
    t = _time_calls(lambda i: op(*sets[i % SETS]), steps, warmup)
    nbytes = B * H * S * D * 10 + B * H * S * 12
    return _hbm("merge", "ring merge step: fp32 acc [1,24,14882,128] updated in place by a bf16 partial + fp32 LSE", nbytes, t, SETS)


def bench_fbcache(dev, steps=30, warmup=60):
    from oracle import fbcache as ofb
    from oracle import inputs

    shape = (1, 32760, 5120)
    prev, cur = inputs.fbcache_pair(shape, seed=1234)
    sets = [(prev.to(dev), cur.to(dev))]
    for i in range(1, SETS):
        sets.append((sets[0][0].roll(i, 1), sets[0][1].roll(i, 1)))  # the same rows in another order
    import torch

    op = torch.ops.para_attn.fbcache_residual_diff
    t = _time_calls(lambda i: op(*sets[i % SETS]), steps, warmup)
    r = _hbm("fbcache", "FBCache residual diff: bf16 [1,32760,5120] pair, threshold 0.12", 4 * prev.numel(), t, SETS)
    ratio = op(*sets[0]).item()
    r["ratio"] = ratio
    r["cache_hit"] = ratio < 0.12
    want = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy())[0]
    if ratio != want:
        raise AssertionError(f"FBCache ratio {ratio} differs from the oracle's {want}")
    r["checked"] = True
    return r


def bench_taylorseer(dev, steps=30, warmup=60):
    import torch

    # cache-hit step with TaylorSeer on: value of 3 stored orders + hidden states, one pass
    shape = (1, 32760, 5120)
    g = torch.Generator(device=dev).manual_seed(5)  # drawn on the device: parity of this kernel is the tests' business
    sets = []
    for _ in range(SETS):
        ds = [torch.randn(shape, generator=g, dtype=torch.bfloat16, device=dev) for _ in range(3)]
        sets.append((ds, torch.randn(shape, generator=g, dtype=torch.bfloat16, device=dev)))
    op = torch.ops.para_attn.taylorseer_value
    t = _time_calls(lambda i: op(sets[i % SETS][0], 2, sets[i % SETS][1]), steps, warmup)
    return _hbm("taylorseer", "TaylorSeer cache hit: 3 stored orders + hidden states, bf16 [1,32760,5120], one pass",
                5 * 2 * sets[0][1].numel(), t, SETS)


def bench_copy(dev, steps=10, warmup=2):
    """Plain device-to-device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    import torch

    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    t = _time_calls(lambda i: dst.copy_(src), steps, warmup)
    r = _hbm("copy", "torch copy_ of 1 GiB (reads 1 GiB, writes 1 GiB)", 2 * n, t, 1)
    r["read_bytes"] = n
    r["write_bytes"] = n
    return r


def bench_yardsticks(dev, steps=30, warmup=60):
    """What plain streaming kernels of the vendor's library reach on this box with the merge step's mix of reads and
    writes, beside which the merge kernel's figure is to be read: HBM efficiency falls with the share of writes
    (bus turn-arounds), so a kernel that reads 6 bytes and writes 4 per element cannot be priced like one that
    only reads.  (1) torch's ``acc.add_(blk)`` on the merge step's operands: fp32 read + 16-bit read + fp32 write
    per element, the same bytes as the merge step less its LSE words, three buffer sets rotated; (2) a 1 GiB copy
    (half reads, half writes).  The read-only end of the scale is the FBCache reduction (``--only fbcache``)."""
    import torch

    B, H, S, D = 1, 24, 14882, 128
    g = torch.Generator(device=dev).manual_seed(1)
    sets = [(torch.randn(B, H, S, D, generator=g, device=dev), torch.randn(B, H, S, D, generator=g, device=dev).bfloat16())
            for _ in range(SETS)]
    out = {}
    t = _time_calls(lambda i: sets[i % SETS][0].add_(sets[i % SETS][1]), steps, warmup)
    out["add_fp32_bf16_in_place"] = _hbm("yardstick", "torch add_: fp32 [1,24,14882,128] += bf16, in place (6 B read, 4 B written per element)",
                                         B * H * S * D * 10, t, SETS)
    del sets
    out["copy_1GiB"] = bench_copy(dev)
    return out


def cpu_baseline(q, k, v):
    """torch's CPU SDPA on the host cores over a bounded sample (about 10-30 s) of the same workload."""
    import torch

    from oracle import attention as oattn

    H, S, D = q.shape[1], q.shape[2], q.shape[3]
    cores = torch.get_num_threads()
    ks, vs = k[:, :1].contiguous(), v[:, :1].contiguous()
    probe = 4096
    oattn.sdpa_lse_torch_cpu(q[:, :1, :512].contiguous(), ks, vs)  # warm the thread pool
    t0 = time.perf_counter()
    oattn.sdpa_lse_torch_cpu(q[:, :1, :probe].contiguous(), ks, vs)
    per_row = (time.perf_counter() - t0) / probe
    # whole heads while they fit in ~20 s, else a leading slice of one head's query rows
    heads = int(min(H, 20.0 / (per_row * S)))
    if heads >= 1:
        qs, kk, vv, rows = q[:, :heads].contiguous(), k[:, :heads].contiguous(), v[:, :heads].contiguous(), S
        what = f"{heads} of {H} heads, all {S} query rows"
    else:
        rows = int(max(probe, 15.0 / per_row))
        heads = 1
        qs, kk, vv = q[:, :1, :rows].contiguous(), ks, vs
        what = f"1 of {H} heads, first {rows} of {S} query rows"
    t0 = time.perf_counter()
    oattn.sdpa_lse_torch_cpu(qs, kk, vv)
    dt = time.perf_counter() - t0
    return {
        "value": round(4.0 * heads * rows * S * D / dt / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"torch CPU SDPA (bf16 out + fp32 LSE): {what} against all {S} keys, {dt:.2f} s",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed calls (default: 20 for the headline, each extra's own otherwise)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed calls before them (default: 30 for the headline)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    singles = {"merge": bench_merge, "fbcache": bench_fbcache, "taylorseer": bench_taylorseer, "sparse": bench_sparse,
               "ring": bench_ring, "flux": bench_flux, "wan": bench_wan, "shapes": bench_shapes, "copy": bench_copy,
               "yardsticks": bench_yardsticks, "wave_rows": bench_wave_rows}
    ap.add_argument("--only", choices=["attn"] + list(singles), default=None,
                    help="profiling aid: run just one kernel's timed loop and print its figures")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (use --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    import paraattention_amd  # noqa: F401
    from paraattention_amd import _lib

    _lib.load()  # no fallback: a missing library is an error
    dev = torch.device("cuda:0")

    if args.only in singles:
        given = {k: v for k, v in (("steps", args.steps), ("warmup", args.warmup)) if v is not None}
        print(json.dumps({args.only: singles[args.only](dev, **given)}))
        return

    steps = 20 if args.steps is None else args.steps
    warmup = 30 if args.warmup is None else args.warmup
    (q, k, v), flops, t, checked = bench_attn(dev, steps, warmup)
    tflops = flops / (t["wall"] * 1e-3) / 1e12
    kern_tflops = flops / (t["mean"] * 1e-3) / 1e12
    result = {
        "metric": "attn TFLOP/s & % bf16 MFMA peak at 119k-token HunyuanVideo shape; ms/call",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(t["wall"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "checked": checked,
        "config": {
            "workload": "HunyuanVideo 720p single-rank Ulysses head share: attention_forward_with_lse "
                        "B=1 H=3 Sq=Skv=119056 D=128 bf16, q/k RMS-normalised, non-causal, out + fp32 LSE",
            "flop_per_call": flops,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "pa::attn_fwd_d128_stream_kernel<pa::BF16, true, 1, false>",
            "achieved": round(kern_tflops, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(kern_tflops / PEAK_BF16_TFLOPS, 4),
            **_ms_fields(t),
            "traffic": TRAFFIC["attn"],
            "traffic_source": TRAFFIC_SOURCE,
        },
    }
    if args.only == "attn":
        print(json.dumps(result))
        return
    if not args.no_extras:
        extras = {"flux_joint_attention": bench_flux(dev)}
        extras.update(bench_ring(dev))
        extras.update(bench_wan(dev))
        extras.update(bench_shapes(dev))
        extras["block_sparse"] = bench_sparse(dev)
        extras["merge_lse"] = bench_merge(dev)
        extras["fbcache_residual_diff"] = bench_fbcache(dev)
        extras["taylorseer_value"] = bench_taylorseer(dev)
        result["extras"] = extras
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(q, k, v)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
