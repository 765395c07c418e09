"""The interception modes route F.scaled_dot_product_attention to the HIP kernels
(src/para_attn/para_attn_interface.py:395-479, src/para_attn/sparse_attn.py:607-640)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import paraattention_amd
from oracle import attention as oattn
from oracle import inputs
from paraattention_amd import interface

pytestmark = pytest.mark.gpu


def test_unified_attn_mode_routes_to_the_kernel(cuda):
    q, k, v = inputs.qkv(1, 3, 200, 333, 128, seed=12)
    ref_out, _ = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    assert interface.kernel_takes(qd, kd, vd)
    direct = torch.ops.para_attn.attention_forward(qd, kd, vd)
    with paraattention_amd.UnifiedAttnMode():
        out = F.scaled_dot_product_attention(qd, kd, vd)
        scaled = F.scaled_dot_product_attention(qd, kd, vd, scale=0.05)
        f32 = F.scaled_dot_product_attention(qd.float(), kd.float(), vd.float())  # not the kernel's: aten
    assert torch.equal(out, direct)  # the same kernel, not aten's
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    assert torch.equal(scaled, torch.ops.para_attn.attention_forward(qd, kd, vd, scale=0.05))
    assert f32.dtype == torch.float32
    np.testing.assert_allclose(f32.cpu().numpy(), ref_out, atol=2e-3, rtol=2e-3)
    with paraattention_amd.config.patch(**{"attention.force_dispatch_to_custom_ops": True}):
        with paraattention_amd.UnifiedAttnMode(attn_func=lambda *a, **kw: "never"):
            assert torch.equal(F.scaled_dot_product_attention(qd, kd, vd), direct)
    # [B,S,H,D] memory, as diffusers hands it over
    qs = qd.transpose(1, 2).contiguous().transpose(1, 2)
    with paraattention_amd.UnifiedAttnMode():
        assert torch.equal(F.scaled_dot_product_attention(qs, kd, vd), direct)


def test_sparse_kv_mode(cuda):
    B, H, Sq, Skv, D = 2, 2, 100, 300, 128
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=13)
    keep = torch.arange(Skv)[None, :] < torch.tensor([300, 177])[:, None]
    ref_out, _ = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep[:, None, None, :].numpy())
    mask = keep[:, None, None, :].expand(B, 1, Sq, Skv).to(cuda)
    with paraattention_amd.SparseKVAttnMode():
        out = F.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    assert torch.equal(out, paraattention_amd.sparse_kv_attn_func(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask))
    with paraattention_amd.SparseKVAttnMode():
        with paraattention_amd.SparseKVAttnMode.disable():
            aten = F.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask)
    np.testing.assert_allclose(aten.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    # under the unified mode a key-only mask goes to the kernel as well
    with paraattention_amd.UnifiedAttnMode():
        out2 = F.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=keep[:, None, None, :].to(cuda))
    assert torch.equal(out2, out)
