"""Argument checks of the Python wrappers that run before anything touches the GPU.

The C ABI takes bare pointers, so an operand shorter than the kernels assume (the LoRA operand
`x @ A` with fewer rows than the activation, a step vector with fewer entries than channels) would
be read out of bounds on the device.  The wrappers must refuse such operands with a ValueError;
these tests pass CPU tensors, so a wrapper that got past its checks would raise the RuntimeError
of `require_gpu` instead."""
import pytest
import torch

import hyclora_amd  # noqa: F401
from hyclora_amd.operators import compress_function as cf
from hyclora_amd.operators import lora_kernels as lk
from hyclora_amd.operators.triton_fuse_lora_silu_hadamard_backward_kernels import triton_fuse_silu_backward
from hyclora_amd.operators.triton_fuse_lora_silu_hadamard_forward_kernels import triton_fuse_silu_forward

BF = torch.bfloat16
B, M, N, R = 2, 8, 64, 16


def t(*shape, dtype=BF):
    return torch.zeros(*shape, dtype=dtype)


def test_well_formed_cpu_operands_reach_the_gpu_check():
    with pytest.raises(RuntimeError, match="GPU only"):
        lk.lora_add(t(B, M, N), t(B, M, R), t(R, N))
    with pytest.raises(RuntimeError, match="GPU only"):
        triton_fuse_silu_forward(t(B, M, R), t(R, N), t(B, M, N), t(1, N), t(B, M, R), t(R, N), t(B, M, N), t(1, N), 4)


@pytest.mark.parametrize("xa_shape", [(B, M - 1, R), (1, M, R), (B, M, R + 4), (B * M * R,)])
def test_lora_add_rejects_a_short_or_misshaped_xa(xa_shape):
    with pytest.raises(ValueError):
        lk.lora_add(t(B, M, N), t(*xa_shape), t(R, N))
    with pytest.raises(ValueError):
        lk.lora_add_quant(t(B, M, N), t(*xa_shape), t(R, N), t(1, N), quantize_bit=4)
    with pytest.raises(ValueError):
        lk.lora_add_restore(t(B, M, N // 2, dtype=torch.uint8), t(1, N), t(*xa_shape), t(R, N), quantize_bit=4)


def test_lora_add_rejects_short_per_channel_vectors_and_other_shapes():
    with pytest.raises(ValueError, match="scale"):
        lk.lora_add_quant(t(B, M, N), t(B, M, R), t(R, N), t(1, N - 32), quantize_bit=4)
    with pytest.raises(ValueError, match="zero point"):
        lk.lora_add_quant(t(B, M, N), t(B, M, R), t(R, N), t(1, N), zero_point=t(1, 8), quantize_bit=4)
    with pytest.raises(ValueError, match="zero point"):
        lk.lora_add_restore(t(B, M, N // 2, dtype=torch.uint8), t(1, N), t(B, M, R), t(R, N), zero_point=t(3),
                            quantize_bit=4)
    with pytest.raises(ValueError, match="width"):
        lk.lora_add(t(B, M, N), t(B, M, R), t(R, N + 32))
    with pytest.raises(ValueError, match="rank"):
        lk.lora_add(t(B, M, N), t(B, M, 2), t(2, N))
    with pytest.raises(ValueError, match="residual"):
        lk.lora_add(t(B, M, N), t(B, M, R), t(R, N), residual=t(B, M - 1, N))
    with pytest.raises(ValueError, match="packed codes"):
        lk.lora_add_restore(t(B, M, N // 4, dtype=torch.uint8), t(1, N), t(B, M, R), t(R, N), quantize_bit=4)


def test_lora_products_reject_short_operands():
    with pytest.raises(ValueError, match="u must be"):
        lk.lora_products(t(B, M, N), u=t(B, M - 1, R))
    with pytest.raises(ValueError, match="v must be"):
        lk.lora_products(t(B, M, N), v=t(R, N - 32))
    with pytest.raises(ValueError, match="u must be"):
        lk.lora_product_from_codes(t(B, M, N // 2, dtype=torch.uint8), t(1, N), t(B, M - 1, R), quantize_bit=4)
    with pytest.raises(ValueError, match="zero point"):
        lk.lora_product_from_codes(t(B, M, N // 2, dtype=torch.uint8), t(1, N), t(B, M, R), zero_point=t(2),
                                   quantize_bit=4)


@pytest.mark.parametrize("bad", ["xa1", "xa2", "s1", "s2", "b2", "rank", "x2"])
def test_fused_kernels_reject_short_operands(bad):
    a = dict(xa1=t(B, M, R), b1=t(R, N), x1=t(B, M, N), s1=t(1, N), xa2=t(B, M, R), b2=t(R, N), x2=t(B, M, N), s2=t(1, N))
    if bad in ("xa1", "xa2"):
        a[bad] = t(B, M - 1, R)
    elif bad in ("s1", "s2"):
        a[bad] = t(1, N - 32)
    elif bad == "b2":
        a[bad] = t(R, N - 32)
    elif bad == "rank":
        a["xa1"], a["b1"], a["xa2"], a["b2"] = t(B, M, 2), t(2, N), t(B, M, 2), t(2, N)
    else:
        a[bad] = t(B, M - 1, N)
    with pytest.raises(ValueError):
        triton_fuse_silu_forward(a["xa1"], a["b1"], a["x1"], a["s1"], a["xa2"], a["b2"], a["x2"], a["s2"], 4)
    if bad != "x2":
        q = t(B, M, N // 2, dtype=torch.uint8)
        with pytest.raises(ValueError):
            triton_fuse_silu_backward(a["xa1"], a["b1"], q, a["s1"], a["xa2"], a["b2"], q, a["s2"], t(B, M, N), 4)


def test_fused_backward_rejects_codes_of_another_shape():
    q = t(B, M, N // 4, dtype=torch.uint8)
    with pytest.raises(ValueError, match="packed codes"):
        triton_fuse_silu_backward(t(B, M, R), t(R, N), q, t(1, N), t(B, M, R), t(R, N), q, t(1, N), t(B, M, N), 4)


def test_channel_list_validation():
    cf.validate_channel_list(torch.tensor([0, 5, 63]), 64)
    cf.validate_channel_list(torch.empty(0, dtype=torch.int64), 64)
    cf.validate_channel_list(None, 64)
    for bad in ([64], [-1], [3, 3]):
        with pytest.raises(ValueError, match="outlier channel"):
            cf.validate_channel_list(torch.tensor(bad), 64)


def test_compressed_map_lists_must_belong_to_the_map():
    from hyclora_amd.operators import softmax_kernels as sk
    g = t(1, 2, 40, 104)                                   # 8320 elements: 3 segments, 4 offsets
    idx, val, seg = torch.zeros(5, dtype=torch.int64), t(5), torch.zeros(4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="GPU only"):
        sk.softmax_backward_from_compressed(idx, val, seg, g)
    for bad in ((idx[:4], val, seg), (idx.int(), val, seg), (idx, val, seg[:3]), (idx, val, seg.int())):
        with pytest.raises(ValueError, match="compressed map|seg_offsets"):
            sk.softmax_backward_from_compressed(*bad, g)
        with pytest.raises(ValueError, match="compressed map|seg_offsets"):
            cf.restore_attention_map(*bad, g.shape)


def test_bf16_vector_is_converted_once_per_tensor_and_again_after_a_change():
    """Frozen per-channel statistics that are not bfloat16 (a zero point kept as a running mean) are converted once
    per tensor object, not at every call; an in-place change of the tensor invalidates the copy."""
    import torch
    from hyclora_amd import _lib
    z = torch.tensor([[1.0, -3.0, 7.5, 0.25]])
    a = _lib.bf16_vector(z)
    assert a.dtype == torch.bfloat16 and a.shape == (4,) and a.tolist() == [1.0, -3.0, 7.5, 0.25]
    assert _lib.bf16_vector(z) is a
    z[0, 1] = 2.0
    b = _lib.bf16_vector(z)
    assert b is not a and b.tolist() == [1.0, 2.0, 7.5, 0.25]
    s = torch.ones(1, 4, dtype=torch.bfloat16)
    assert _lib.bf16_vector(s).data_ptr() == s.data_ptr()          # already bfloat16: a view, nothing kept
    n = len(_lib._BF16_VECTORS)
    del z, a, b
    import gc
    gc.collect()
    assert len(_lib._BF16_VECTORS) == n - 1
