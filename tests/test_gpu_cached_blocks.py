"""CachedTransformerBlocks (src/para_attn/first_block_cache/utils.py:333-451) over toy blocks whose arithmetic
is exact on both devices (multiplies, adds and rolls in bf16), against a plain restatement of the reference's
step on the CPU with torch's eager ops: same hit/miss sequence, same outputs bit for bit."""
import pytest
import torch

from paraattention_amd import fbcache

pytestmark = pytest.mark.gpu


class Dual(torch.nn.Module):
    def __init__(self, i, first=True, only=False):
        super().__init__()
        self.a, self.b, self.shift, self.first, self.only = 0.5 + 0.125 * i, 0.25, i + 1, first, only

    def forward(self, h, e, scale=1.0):
        h2 = h * self.a + torch.roll(h, self.shift, 1) * (self.b * scale)
        if self.only:
            return h2
        e2 = e * 0.75 + torch.roll(e, self.shift, 1) * 0.125
        return (h2, e2) if self.first else (e2, h2)


class Single(torch.nn.Module):
    def __init__(self, i):
        super().__init__()
        self.shift = i + 2

    def forward(self, x, scale=1.0):
        return x * 0.875 + torch.roll(x, self.shift, 1) * (0.0625 * scale)


def reference_steps(duals, singles, steps, *, threshold, warmup, first=True, only=False, scale=1.0):
    """The reference's forward (utils.py:349-394) with torch eager ops on the CPU."""
    prev_first = res = enc_res = None
    outs, hits = [], []

    def run(block, h, e):
        out = block(h, e, scale=scale)
        if isinstance(out, torch.Tensor):
            return out, e
        return out if first else (out[1], out[0])

    for t, (h, e) in enumerate(steps):
        orig = h
        h, e = run(duals[0], h, e)
        first_res = h - orig
        hit = False
        if t >= warmup and threshold > 0 and prev_first is not None:
            diff = (prev_first - first_res).abs().mean() / prev_first.abs().mean()
            hit = diff.item() < threshold
        if hit:
            h = res + h
            if not only:
                e = enc_res + e
        else:
            prev_first = first_res
            h0, e0 = h, e
            for blk in duals[1:]:
                h, e = run(blk, h, e)
            if singles is not None:
                x = torch.cat([e, h], dim=1)
                for blk in singles:
                    x = blk(x, scale=scale)
                e, h = x.split([e.shape[1], x.shape[1] - e.shape[1]], dim=1)
            res, enc_res = h - h0, e - e0
        outs.append((h, e))
        hits.append(hit)
    return outs, hits


def make_steps(n, seed):
    g = torch.Generator().manual_seed(seed)
    base_h, base_e = torch.randn(2, 48, 64, generator=g), torch.randn(2, 12, 64, generator=g)
    steps = []
    for t in range(n):
        jump = 1.0 if t in (4, 5) else 0.02  # two steps that move too much to reuse the cache
        base_h = base_h + jump * torch.randn(base_h.shape, generator=g)
        steps.append((base_h.bfloat16(), base_e.bfloat16()))
    return steps


@pytest.mark.parametrize("with_singles,first,only", [(True, True, False), (False, False, False), (False, True, True)])
def test_cached_blocks_follow_the_reference_step(cuda, with_singles, first, only):
    duals = [Dual(i, first, only) for i in range(4)]
    singles = [Single(i) for i in range(2)] if with_singles else None
    steps = make_steps(9, seed=3)
    ref_outs, ref_hits = reference_steps(duals, singles, steps, threshold=0.1, warmup=1, first=first, only=only, scale=0.5)
    assert any(ref_hits) and not all(ref_hits[2:]), ref_hits  # the sequence has both outcomes after warm-up

    mod = fbcache.CachedTransformerBlocks(torch.nn.ModuleList(duals), torch.nn.ModuleList(singles) if singles else None,
                                          return_hidden_states_first=first, return_hidden_states_only=only)
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.1, warmup_steps=1)
    hits = []
    with fbcache.cache_context(ctx):
        for t, (h, e) in enumerate(steps):
            had = ctx.get_buffer("first_hidden_states_residual")
            out = mod(h.to(cuda), e.to(cuda), scale=0.5)
            hits.append(ctx.get_buffer("first_hidden_states_residual") is had and t > 0)
            if only:
                got_h, got_e = out, None
            else:
                got_h, got_e = out if first else (out[1], out[0])
            assert torch.equal(got_h.cpu(), ref_outs[t][0]), f"step {t}: hidden states differ"
            if got_e is not None:
                assert torch.equal(got_e.cpu(), ref_outs[t][1]), f"step {t}: encoder hidden states differ"
    assert hits == ref_hits


def test_skip_layer_guidance_drops_blocks(cuda):
    """utils.py:102-114, 407-428: on the alternating pass inside the step window the listed blocks are not run."""
    calls = []

    class Counting(Dual):
        def forward(self, h, e, scale=1.0):
            calls.append(self.shift - 1)
            return super().forward(h, e, scale)

    duals = [Counting(i) for i in range(4)]
    mod = fbcache.CachedTransformerBlocks(torch.nn.ModuleList(duals))
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.0, enable_alter_cache=True, slg_layers=[2],
                                       slg_start=0.0, slg_end=0.5, num_inference_steps=4)
    h, e = (t.to(cuda) for t in make_steps(1, seed=1)[0])
    seen = []
    with fbcache.cache_context(ctx):
        for _ in range(6):  # passes alternate: plain, alter, plain, alter, ...
            calls.clear()
            mod(h, e)
            seen.append(list(calls))
    # steps 0 and 1 lie in [0, 2): their alternating passes (2nd and 4th call) skip block 2; step 2 does not
    assert seen == [[0, 1, 2, 3], [0, 1, 3], [0, 1, 2, 3], [0, 1, 3], [0, 1, 2, 3], [0, 1, 2, 3]]
