"""Host layer without a GPU: op names and schemas equal the reference's, fake (meta) implementations give
the reference's output contract, config flags, cache-context gates and the no-fallback rule."""
import os

import pytest
import torch

import paraattention_amd
from paraattention_amd import config, fbcache, ops

SDPA_SCHEMA = (
    "(Tensor query, Tensor key, Tensor value, Tensor? attn_mask=None, float dropout_p=0., "
    "bool is_causal=False, *, float? scale=None)"
)


def test_op_schemas_match_reference():
    # src/para_attn/ops/__init__.py:160-179, 204-223, 302-321: names, argument order, defaults, keyword-only scale
    assert str(torch.ops.para_attn.attention_forward_with_lse.default._schema) == (
        "para_attn::attention_forward_with_lse" + SDPA_SCHEMA + " -> (Tensor, Tensor)"
    )
    assert str(torch.ops.para_attn.attention_forward.default._schema) == "para_attn::attention_forward" + SDPA_SCHEMA + " -> Tensor"
    assert str(torch.ops.para_attn.attention_forward_sparse_kv.default._schema) == (
        "para_attn::attention_forward_sparse_kv" + SDPA_SCHEMA + " -> Tensor"
    )
    for name in ("merge_attention_lse", "merge_attention_lse_", "attention_forward_block_sparse", "fbcache_residual_diff",
                 "fbcache_first_residual_diff", "fbcache_apply_residual"):
        assert hasattr(torch.ops.para_attn, name)
    assert torch.ops.para_attn.merge_attention_lse_.default._schema.arguments[0].alias_info.is_write


def test_fake_impls_give_reference_contract():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        q = torch.empty(2, 24, 4096, 128, dtype=torch.bfloat16, device="cuda")
        k = torch.empty(2, 24, 1024, 128, dtype=torch.bfloat16, device="cuda")
        out, lse = torch.ops.para_attn.attention_forward_with_lse(q, k, k)
        # the reference's own assertions (tests/ops/test_ops.py:63-64)
        assert out.shape == (2, 24, 4096, 128) and out.dtype == torch.bfloat16
        assert lse.shape == (2, 24, 4096) and lse.dtype == torch.float32
        assert torch.ops.para_attn.attention_forward(q, k, k).shape == q.shape
        assert torch.ops.para_attn.attention_forward_sparse_kv(q, k, k).shape == q.shape
        mo, ml = torch.ops.para_attn.merge_attention_lse(out, lse, out, lse)
        assert mo.dtype == torch.float32 and mo.shape == out.shape and ml.shape == lse.shape
        mo, _ = torch.ops.para_attn.merge_attention_lse(out, lse, out, lse, torch.bfloat16)
        assert mo.dtype == torch.bfloat16
        bm = torch.empty(32, 8, dtype=torch.bool, device="cuda")
        so, sl = torch.ops.para_attn.attention_forward_block_sparse(q, k, k, bm)
        assert so.shape == q.shape and sl.shape == (2, 24, 4096)
        r = torch.ops.para_attn.fbcache_residual_diff(q, q)
        assert r.shape == () and r.dtype == torch.bfloat16


def test_fake_outputs_keep_the_query_layout():
    """The real ops write the output in the query's memory layout (ops._out_like); the fakes must describe the same
    strides or a compiled consumer is planned against the wrong ones.  The GPU suite compares fake and real with
    torch.library.opcheck; here the rule itself is pinned without a device."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    ns = torch.ops.para_attn
    with FakeTensorMode():
        bshd = torch.empty(2, 200, 3, 128, dtype=torch.bfloat16, device="cuda").transpose(1, 2)
        assert bshd.stride() == (76800, 128, 384, 1)
        bm = torch.empty(3, 2, 4, dtype=torch.bool, device="cuda")
        runs = ns.block_sparse_key_runs(bm, 200)
        outs = [
            ns.attention_forward_with_lse(bshd, bshd, bshd)[0],
            ns.attention_forward(bshd, bshd, bshd),
            ns.attention_forward_sparse_kv(bshd, bshd, bshd),
            ns.attention_forward_sweep(bshd, [bshd], [bshd])[0],
            ns.attention_forward_block_sparse(bshd, bshd, bshd, bm)[0],
            ns.attention_forward_block_sparse_runs(bshd, bshd, bshd, runs, 3, 2, 4)[0],
        ]
        for o in outs:
            assert o.shape == bshd.shape and o.stride() == bshd.stride()
        assert ns.attention_forward_with_lse(bshd, bshd, bshd)[1].stride() == (600, 200, 1)
        # rows the kernels cannot write in place (row stride not a multiple of 8 elements; head_dim not innermost)
        ragged = torch.empty(2, 3, 200, 132, dtype=torch.bfloat16, device="cuda")[..., :128]
        assert ns.attention_forward(ragged, ragged, ragged).is_contiguous()
        dfirst = torch.empty(2, 3, 128, 200, dtype=torch.bfloat16, device="cuda").transpose(2, 3)
        assert ns.attention_forward(dfirst, dfirst, dfirst).is_contiguous()
        # the key-range buffer: the library's own size for the mask geometry, single and paired layouts
        lib = paraattention_amd._lib.load()
        for hm, nq, nk in ((1, 2, 64), (3, 2, 4), (24, 256, 256)):
            words = ns.block_sparse_key_runs(torch.empty(hm, nq, nk, dtype=torch.bool, device="cuda"), nk * 128).numel()
            assert words * 4 >= lib.pa_blocksparse_workspace_bytes(hm, nq, nk) > (words - 1) * 4


def test_operands_of_another_device_stop_before_any_launch():
    """The op bodies, called directly with the query on one device ("meta": no memory, so nothing can be launched
    from it) and another operand on the CPU: every one of them raises the device error first.  A CPU mask beside
    GPU activations reaches the GPU implementation (the dispatcher picks it for the mixed call), where its pointer
    would be read by a kernel."""
    bf = torch.bfloat16
    q = torch.empty(2, 2, 64, 128, dtype=bf, device="meta")
    cq = torch.empty(2, 2, 64, 128, dtype=bf)
    keep = torch.ones(2, 1, 1, 64, dtype=torch.bool)
    lse, clse = torch.empty(2, 2, 64, device="meta"), torch.empty(2, 2, 64)
    acc, cacc = torch.empty(2, 2, 64, 128, device="meta"), torch.empty(2, 2, 64, 128)
    bm = torch.ones(2, 2, dtype=torch.bool)
    h, ch = torch.empty(4, 64, dtype=bf, device="meta"), torch.empty(4, 64, dtype=bf)
    calls = [
        (ops.attention_forward_with_lse, (q, q, q, keep)),
        (ops.attention_forward_with_lse, (q, q, q, keep.float())),
        (ops.attention_forward_with_lse, (q, cq, q)),
        (ops.attention_forward_with_lse, (q, q, cq)),
        (ops.attention_forward, (q, q, q, keep)),
        (ops.attention_forward, (q, cq, cq)),
        (ops.attention_forward_sparse_kv, (q, q, q, keep)),
        (ops.attention_forward_sparse_kv, (q, q, cq)),
        (ops.merge_attention_lse, (acc, clse, q, lse)),
        (ops.merge_attention_lse, (acc, lse, cq, lse)),
        (ops.merge_attention_lse, (acc, lse, q, clse)),
        (ops.merge_attention_lse_, (acc, lse, cq, lse)),
        (ops.attention_forward_accumulate_, (cacc, lse, q, q, q)),
        (ops.attention_forward_accumulate_, (acc, clse, q, q, q)),
        (ops.attention_forward_accumulate_, (acc, lse, q, cq, q)),
        (ops.attention_forward_accumulate_final, (acc, clse, q, q, q)),
        (ops.attention_forward_sweep, (q, [q, cq], [q, q])),
        (ops.attention_forward_sweep, (q, [q, q], [cq, q])),
        (ops.attention_forward_block_sparse, (q, q, q, bm)),
        (ops.attention_forward_block_sparse, (q, cq, q, bm.to("meta"))),
        (ops.attention_forward_block_sparse_runs, (q, q, q, torch.zeros(64, dtype=torch.int32), 1, 2, 2)),
        (ops.fbcache_residual_diff, (h, ch)),
        (ops.fbcache_first_residual_diff, (h, ch)),
        (ops.fbcache_first_residual_diff, (h, h, ch)),
        (ops.fbcache_apply_residual, (ch, h)),
        (ops.taylorseer_derivatives, (h, [h, ch], 2.0)),
        (ops.taylorseer_value, ([h, ch], 2)),
        (ops.taylorseer_value, ([h, h], 2, ch)),
    ]
    for op, args in calls:
        with pytest.raises(ValueError, match="device"):
            op._init_fn(*args)


def test_cpu_tensors_are_refused_not_emulated():
    # the reference asserts "Must be CUDA tensors" (src/para_attn/ops/__init__.py:123); here the dispatcher refuses
    q = torch.randn(1, 1, 16, 128).bfloat16()
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.attention_forward_with_lse(q, q, q)
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.fbcache_residual_diff(q, q)
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.merge_attention_lse(q.float(), q[..., 0].float(), q, q[..., 0].float())


def test_product_does_not_import_the_oracle():
    pkg = os.path.dirname(paraattention_amd.__file__)
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f


def test_config_flags_and_patch():
    assert config.attention.allow_reduced_precision_compute in (False, True)
    before = config.attention.allow_reduced_precision_compute
    with config.patch(**{"attention.allow_reduced_precision_compute": not before}):
        assert config.attention.allow_reduced_precision_compute is (not before)
    assert config.attention.allow_reduced_precision_compute is before
    with pytest.raises(AttributeError):
        with config.patch(**{"attention.no_such_flag": True}):
            pass


def test_cache_context_gates_need_no_device():
    x = torch.zeros(1, 4, 8)
    with pytest.raises(AssertionError):
        fbcache.get_can_use_cache(x)  # no context set (first_block_cache/utils.py:196-201)
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.0)
    with fbcache.cache_context(ctx):
        ctx.mark_step_begin()
        assert fbcache.get_can_use_cache(x) is False  # threshold gate, utils.py:273-275
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.1, warmup_steps=2)
    with fbcache.cache_context(ctx):
        ctx.mark_step_begin()
        assert ctx.get_current_step() == 0 and ctx.is_in_warmup()
        assert fbcache.get_can_use_cache(x) is False  # warm-up gate, utils.py:271
        ctx.mark_step_begin(); ctx.mark_step_begin()
        assert not ctx.is_in_warmup()
        assert fbcache.get_can_use_cache(x) is False  # nothing stored yet, utils.py:280
    assert fbcache.get_current_cache_context() is None
    assert fbcache.are_two_tensors_similar(x, x, threshold=0.0) is False
    assert fbcache.are_two_tensors_similar(x, x[:, :2], threshold=0.5) is False
    # alternating (cond / uncond) cache: buffer names and thresholds switch (utils.py:54-72, 83-92)
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.1, alter_residual_diff_threshold=0.2, enable_alter_cache=True)
    ctx.mark_step_begin()
    assert ctx.is_alter_cache is False and ctx.executed_steps == 1 and ctx.get_residual_diff_threshold() == 0.1
    ctx.set_buffer("first_hidden_states_residual", 1)
    ctx.mark_step_begin()
    assert ctx.is_alter_cache is True and ctx.executed_steps == 1 and ctx.get_residual_diff_threshold() == 0.2
    assert ctx.get_buffer("first_hidden_states_residual") is None
    ctx.set_buffer("first_hidden_states_residual", 2)
    assert ctx.buffers == {"first_hidden_states_residual": 1, "first_hidden_states_residual_alter": 2}


def test_row_view_helper():
    t = torch.zeros(2, 300, 512)
    assert ops._as_rows(t) == (600, 512, 512, 1)
    assert ops._as_rows(t[..., ::4]) == (600, 128, 512, 4)
    assert ops._as_rows(t[:, ::2]) is None or ops._as_rows(t[:, ::2])[0] == 300  # rows no longer collapse to one stride
    assert ops._as_rows(torch.zeros(())) == (1, 1, 1, 1)
    assert ops._as_rows(t.transpose(0, 1)) is None


def test_mask_broadcasting_follows_torch():
    """attn_mask is read as F.scaled_dot_product_attention reads it (trailing dimensions aligned with
    [B,H,Sq,Skv], src/para_attn/ops/__init__.py:215-223): a 2-D mask is [Sq,Skv], never a per-batch key mask."""
    from paraattention_amd import _lib

    B, H, Sq, Skv = 2, 3, 5, 10
    m = torch.rand(B, Skv) < 0.5
    t, kind, st = ops._broadcast_mask(m[:, None, None, :], B, H, Sq, Skv, torch.bfloat16)
    assert kind == _lib.PA_MASK_BOOL and list(st) == [Skv, 0, 0, 1]
    t, kind, st = ops._broadcast_mask(torch.zeros(Sq, Skv), B, H, Sq, Skv, torch.bfloat16)
    assert kind == _lib.PA_MASK_F32 and list(st) == [0, 0, Skv, 1] and t.shape == (1, 1, Sq, Skv)
    t, kind, st = ops._broadcast_mask(torch.zeros(H, 1, Skv, dtype=torch.bfloat16), B, H, Sq, Skv, torch.bfloat16)
    assert kind == _lib.PA_MASK_ACT and list(st) == [0, Skv, 0, 1]
    t, kind, st = ops._broadcast_mask(torch.zeros(B, H, Sq, Skv, dtype=torch.float16), B, H, Sq, Skv, torch.bfloat16)
    assert kind == _lib.PA_MASK_F32 and t.dtype == torch.float32  # another float type than the activations': widened
    with pytest.raises(ValueError):
        ops._broadcast_mask(m, B, H, Sq, Skv, torch.bfloat16)  # [2,10] against Sq = 5: does not broadcast
    with pytest.raises(ValueError):
        ops._broadcast_mask(torch.zeros(Sq, Skv, dtype=torch.int32), B, H, Sq, Skv, torch.bfloat16)
    with pytest.raises(ValueError):
        ops._broadcast_mask(torch.zeros(1, 1, 1, 1, Skv), B, H, Sq, Skv, torch.bfloat16)


def test_merger_refuses_partial_mode():
    m = paraattention_amd.SDPAMerger(True, 2)
    with pytest.raises(NotImplementedError):
        m.step(torch.zeros(1, 1, 4, 8), torch.zeros(1, 1, 4), partial=True)


def test_cache_context_builds_taylorseers():
    """utils.py:39-43, 90-97: one TaylorSeer, or two with the alternating cache; mark_step_begin advances the active one."""
    from paraattention_amd import fbcache
    from paraattention_amd.taylorseer import TaylorSeer

    ctx = fbcache.create_cache_context(enable_taylorseer=True, taylorseer_kwargs={"n_derivatives": 1, "warmup_steps": 2})
    assert isinstance(ctx.taylorseer, TaylorSeer) and ctx.alter_taylorseer is None and ctx.taylorseer.ORDER == 2
    ctx.mark_step_begin()
    ctx.mark_step_begin()
    assert ctx.taylorseer.current_step == 1 and ctx.get_taylorseer() is ctx.taylorseer
    ctx = fbcache.create_cache_context(enable_taylorseer=True, enable_alter_cache=True)
    assert ctx.alter_taylorseer is not None
    ctx.mark_step_begin()  # -> not alter: the plain one advances
    assert ctx.get_taylorseer() is ctx.taylorseer and ctx.taylorseer.current_step == 0 and ctx.alter_taylorseer.current_step == -1
    ctx.mark_step_begin()  # -> alter
    assert ctx.get_taylorseer() is ctx.alter_taylorseer and ctx.alter_taylorseer.current_step == 0
    assert fbcache.create_cache_context().taylorseer is None


def test_taylorseer_schedule_and_limits():
    """taylorseer.py:21-27 (schedule) with the reference's own self-test settings; the kernels take at most 4 orders."""
    import pytest

    from paraattention_amd.taylorseer import TaylorSeer

    ts = TaylorSeer(n_derivatives=2, warmup_steps=2, skip_interval_steps=2)
    assert [ts.should_compute_full(s) for s in range(8)] == [True, True, False, True, False, True, False, True]
    assert TaylorSeer(compute_step_map=[False, True]).should_compute_full(1) is True
    assert ts.approximate_value() == 0  # nothing stored: the reference's empty sum
    with pytest.raises(NotImplementedError):
        TaylorSeer(n_derivatives=5)


def test_unified_attn_mode_on_cpu_passes_through():
    """Calls the kernel does not take (CPU tensors here) reach F.scaled_dot_product_attention untouched, through
    all three stages (para_attn_interface.py:445-475); a mesh of several ranks is refused."""
    import torch
    import torch.nn.functional as F

    import paraattention_amd
    from paraattention_amd import interface

    q, k, v = (torch.randn(1, 2, 8, 16) for _ in range(3))
    want = F.scaled_dot_product_attention(q, k, v)
    with paraattention_amd.UnifiedAttnMode():
        got = F.scaled_dot_product_attention(q, k, v)
        assert torch.equal(torch.add(q, 1), q + 1)  # other functions are left alone
    assert torch.equal(got, want)
    calls = []
    with paraattention_amd.UnifiedAttnMode(attn_func=lambda *a, **kw: calls.append((a, kw)) or "mine"):
        assert F.scaled_dot_product_attention(q, k, v, scale=0.5) == "mine"
    assert len(calls) == 1 and calls[0][1] == {"scale": 0.5}
    with paraattention_amd.UnifiedAttnMode(skip_small_kv=True, attn_func=lambda *a, **kw: "mine"):
        assert F.scaled_dot_product_attention(q, k[:, :, :4], v[:, :, :4]) is not "mine"  # more queries than keys: skipped
        assert F.scaled_dot_product_attention(q[:, :, :4], k, v) == "mine"
    with paraattention_amd.UnifiedAttnMode(attn_func=lambda *a, **kw: "mine"):
        with paraattention_amd.UnifiedAttnMode.disable():
            assert torch.equal(F.scaled_dot_product_attention(q, k, v), want)
    assert not interface.kernel_takes(q, k, v)

    class FakeMesh:
        def size(self):
            return 8

    import pytest

    with pytest.raises(NotImplementedError):
        paraattention_amd.UnifiedAttnMode(FakeMesh())


def test_skip_layer_guidance_window():
    """utils.py:102-114: only on the alternating pass, only for listed blocks, only inside [start, end) of the schedule."""
    from paraattention_amd import fbcache

    ctx = fbcache.create_cache_context(slg_layers=[1, 3], enable_alter_cache=True, num_inference_steps=10, slg_start=0.1, slg_end=0.3)
    assert ctx.is_slg_enabled() and not fbcache.create_cache_context().is_slg_enabled()
    seen = []
    for _ in range(10):  # plain / alter passes of steps 0..4
        ctx.mark_step_begin()
        seen.append((ctx.get_current_step(), ctx.is_alter_cache, ctx.slg_should_skip_block(1), ctx.slg_should_skip_block(2)))
    assert seen == [(0, False, False, False), (0, True, False, False), (1, False, False, False), (1, True, True, False),
                    (2, False, False, False), (2, True, True, False), (3, False, False, False), (3, True, False, False),
                    (4, False, False, False), (4, True, False, False)]
    whole = fbcache.create_cache_context(slg_layers=[1], enable_alter_cache=True, num_inference_steps=10, slg_start=0.0, slg_end=1.0)
    whole.mark_step_begin()
    whole.mark_step_begin()
    assert whole.is_alter_cache and not whole.slg_should_skip_block(1)  # the degenerate window switches it off (utils.py:107-108)


def test_cache_context_module_level_accessors():
    """The module-level accessors of the reference (first_block_cache/utils.py:124-190, 263-267) read the current
    context, respect the alternating cache's "_alter" buffer names and refuse to run without a context."""
    with pytest.raises(AssertionError):
        fbcache.get_buffer("x")
    ctx = fbcache.create_cache_context(residual_diff_threshold=torch.tensor(0.12), alter_residual_diff_threshold=0.2,
                                       enable_alter_cache=True, warmup_steps=2, downsample_factor=4)
    with fbcache.cache_context(ctx):
        assert fbcache.get_downsample_factor() == 4
        # is_alter_cache starts True (utils.py:37): the alternating threshold and the "_alter" names apply
        assert fbcache.get_residual_diff_threshold() == 0.2
        fbcache.set_buffer("h", 1)
        assert ctx.buffers == {"h_alter": 1} and fbcache.get_buffer("h") == 1
        fbcache.mark_step_begin()  # flips to the main pass and counts a step
        assert fbcache.get_residual_diff_threshold() == pytest.approx(0.12) and isinstance(fbcache.get_residual_diff_threshold(), float)
        assert fbcache.get_buffer("h") is None
        fbcache.set_buffer("h", 2)
        fbcache.remove_buffer("h")
        fbcache.remove_buffer("h")  # absent: no error (utils.py:74-78)
        assert ctx.buffers == {"h_alter": 1}
        assert fbcache.is_in_warmup()          # step 0 of 2 warm-up steps
        for _ in range(4):
            fbcache.mark_step_begin()          # two more counted steps
        assert ctx.get_current_step() == 2 and not fbcache.is_in_warmup()
    assert fbcache.get_current_cache_context() is None
    # incremental names count per name from 0 (utils.py:45-53)
    assert [ctx.get_incremental_name(), ctx.get_incremental_name(), ctx.get_incremental_name("a")] == ["default_0", "default_1", "a_0"]
    ctx.reset_incremental_names()
    assert ctx.get_incremental_name() == "default_0"
