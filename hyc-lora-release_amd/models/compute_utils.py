"""Torch-side glue of the fused layers (reference: models/utils/compute_utils.py:7-51 and
operators/rope_kernels.py:81-126).  The frozen-weight GEMMs and the attention products are library /
torch operations in the reference as well; only what surrounds them is compressed.  RoPE is the
in-place HIP kernel of operators/rope_kernels.py, re-exported here."""
import torch

from ..operators import lora_kernels
from ..operators.nf4 import dequantize_nf4


def hidden_to_head_shape(x: torch.Tensor, num_heads: int):
    bsz, seq_len, hidden = x.shape
    return x.reshape(bsz, seq_len, num_heads, hidden // num_heads).transpose(1, 2)


def head_to_hidden_shape(x: torch.Tensor):
    bsz, _, seq_len, _ = x.shape
    return x.transpose(1, 2).reshape(bsz, seq_len, -1).contiguous()


_MAX_BATCH_LOOP = 16


def heads_matmul(a: torch.Tensor, b: torch.Tensor, out_hidden: bool = False):
    """a @ b for [B, H, M, K] x [B, H, K, N] operands that are *views* of hidden-layout tensors
    ([B, S, H*D] seen as [B, H, S, D]).  torch.matmul would first copy such a view into head-major
    memory (the reference pays that copy at every attention product); a batched GEMM over the heads
    of one batch element reads it in place (row stride H*D, batch stride D), so this loops over the
    batch.  out_hidden=True writes the result [B, H, M, N] into a hidden-layout buffer and returns
    its [B, H, M, N] view, which makes the following head_to_hidden_shape free."""
    B, H, M, _ = a.shape
    N = b.shape[-1]
    if B > _MAX_BATCH_LOOP or not a.is_cuda or a.dtype != b.dtype:
        r = torch.matmul(a, b)
        return r.transpose(1, 2).contiguous().transpose(1, 2) if out_hidden else r
    if out_hidden:
        out = a.new_empty(B, M, H, N).transpose(1, 2)
    else:
        out = a.new_empty(B, H, M, N)
    for i in range(B):
        torch.bmm(a[i], b[i], out=out[i])
    return out


def dense_weight(w: torch.Tensor, quant_state):
    """Frozen weight as a dense [out, in] matrix.  quant_state None = already dense (the benchmark
    configurations); otherwise a bitsandbytes-format NF4 weight, dequantised by the HIP kernel (the
    reference calls BF.dequantize_nf4 at the same place, compute_utils.py:19, :29)."""
    if quant_state is None:
        return w
    return dequantize_nf4(w, quant_state)


def lora_forward(w, w_quant_state, w_lora_a, w_lora_b, b, x, residual=None, x_lora_a=None):
    """-> (x @ W^T [+ b] + (x @ A) @ B, the frozen part alone, x @ A).  Reference :18-25.  The LoRA
    product and the add are one MFMA kernel over the frozen part (bf16 operands); other dtypes
    take the torch expression.  `residual` (not in the reference's signature) is added to the first
    result in the same pass - the `x + o_final` that follows the projection in the layers.
    `x_lora_a`: x @ A where the producer of x has already formed it."""
    x_main, x_lora_a = lora_parts(w, w_quant_state, w_lora_a, b, x, x_lora_a)
    w_lora_b = w_lora_b.to(x_main.dtype)
    if lora_kernels.supported(x_main, x_lora_a, w_lora_b) and (residual is None or residual.dtype == x_main.dtype):
        return lora_kernels.lora_add(x_main, x_lora_a, w_lora_b, residual=residual), x_main, x_lora_a
    y = x_main + x_lora_a @ w_lora_b
    return (y if residual is None else residual + y), x_main, x_lora_a


def lora_parts(w, w_quant_state, w_lora_a, b, x, x_lora_a=None):
    """-> (x @ W^T [+ b], x @ A): what lora_forward computes before the LoRA add.  x @ A is taken
    from `x_lora_a` when the caller has it already (the fused norm kernel forms it)."""
    wt = dense_weight(w, w_quant_state).t()
    x = x.to(wt.dtype)
    x_main = x @ wt
    if b is not None:
        x_main = x_main + b.to(wt.dtype)
    if x_lora_a is None:
        x_lora_a = x @ w_lora_a.to(wt.dtype)
    return x_main, x_lora_a.to(wt.dtype)


def lora_backward(w, w_quant_state, w_lora_a, w_lora_b, x, x_lora_a, grad_y, x_codes=None, accumulate=None,
                  defer_input=False):
    """-> (grad lora_A, grad lora_B, grad x).  Reference :28-36.

    With bf16 operands the rank-R products stream their wide operand once on the matrix cores:
    grad_y gives `grad_y @ B^T` and `xa^T @ grad_y` in one pass, and `x^T @ grad_medium` is taken
    from x - or straight from its packed codes `x_codes = (q, scale, zero_point or None, q_bit)`,
    in which case x may be None and is never dequantised.  Those results are summed over the batch in
    fp32 and have the parameters' shapes; the torch expressions below return one gradient per batch
    element, as the reference does, and leave the sum to autograd.  `accumulate`, a running sum of
    input gradients, is added to grad x in the pass that adds its LoRA part (`grad_x += grad_x_temp`
    in the layers) and may be overwritten.  With `defer_input` the third result is not grad x but its
    two terms and the operand that joins them, `(grad_y @ W, grad_y @ B^T, A^T)`, for lora_input_sum, which
    adds up the input gradients of projections that share their input in one pass."""
    wd = dense_weight(w, w_quant_state)          # [out, in]
    dt = wd.dtype
    grad_y = grad_y.to(dt)
    w_lora_a, w_lora_b = w_lora_a.to(dt), w_lora_b.to(dt)
    r = w_lora_b.shape[0]
    if lora_kernels.contract_supported(grad_y, grad_y.shape[-1], r) and x_lora_a.dtype == dt:
        # xa^T @ grad_y written as [N, R], the layout of the lora_B weight this gradient ends up in: what is
        # returned is its [R, N] view, and autograd's transpose back is then contiguous and stored without a copy
        grad_b, grad_mid = lora_kernels.lora_products(grad_y, u=x_lora_a, v=w_lora_b, p1_transposed=True)
        grad_b = grad_b.t()
    else:
        grad_mid = grad_y @ w_lora_b.mT
        grad_b = x_lora_a.to(dt).mT @ grad_y
    if x_codes is not None and lora_kernels.contract_supported(grad_mid, w_lora_a.shape[0], r):
        q, scale, zero_point, q_bit = x_codes
        grad_a = lora_kernels.lora_product_from_codes(q, scale, grad_mid, zero_point, q_bit).t()
    else:
        if x is None:
            from ..operators.compress_function import (decompression_dequantization,
                                                       decompression_dequantization_with_zero_point)
            q, scale, zero_point, q_bit = x_codes
            x = decompression_dequantization(q, scale, q_bit) if zero_point is None else \
                decompression_dequantization_with_zero_point(q, scale, zero_point, q_bit)
        if lora_kernels.contract_supported(x, x.shape[-1], r) and grad_mid.dtype == x.dtype:
            grad_a = lora_kernels.lora_products(x, u=grad_mid)[0].t()
        else:
            grad_a = x.to(dt).mT @ grad_mid
    grad_x = grad_y @ wd
    if defer_input:
        return grad_a, grad_b, (grad_x, grad_mid, w_lora_a.mT)
    if lora_kernels.supported(grad_x, grad_mid, w_lora_a.mT) and (accumulate is None or accumulate.dtype == dt):
        grad_x = lora_kernels.lora_add(grad_x, grad_mid, w_lora_a.mT, inplace=True, residual=accumulate)
    else:
        grad_x += grad_mid @ w_lora_a.mT
        if accumulate is not None:
            grad_x = accumulate + grad_x
    return grad_a, grad_b, grad_x


def lora_input_sum(parts):
    """Sum of the input gradients of projections that share their input, from the deferred terms lora_backward
    returns: acc = t_0; acc += t_1; ... with t_i = (grad_y @ W)_i + (grad_y @ B^T)_i @ A_i^T, every operation
    rounded as the chain of lora_backward(..., accumulate=acc) calls rounds it (the reference's
    `grad_x += grad_x_temp`).  Two or three bf16 terms of rank <= 16 take one pass over their operands."""
    terms = list(parts)
    if lora_kernels.supported_sum(terms):
        return lora_kernels.lora_add_sum(terms)
    acc = None
    for grad_x, grad_mid, a_t in terms:
        if lora_kernels.supported(grad_x, grad_mid, a_t) and (acc is None or acc.dtype == grad_x.dtype):
            acc = lora_kernels.lora_add(grad_x, grad_mid, a_t, inplace=True, residual=acc)
        else:
            grad_x += grad_mid @ a_t
            acc = grad_x if acc is None else acc + grad_x
    return acc


def repeat_kv(hidden_states: torch.Tensor, n_rep: int):
    """[B, KV, S, D] -> [B, KV * n_rep, S, D], every key / value head n_rep times in a row.  Reference :38-43."""
    if n_rep == 1:
        return hidden_states
    b, kv, s, d = hidden_states.shape
    return hidden_states[:, :, None, :, :].expand(b, kv, n_rep, s, d).reshape(b, kv * n_rep, s, d)


def repeat_kv_backward(grad_output: torch.Tensor, n_rep: int):
    """Gradient of repeat_kv: the n_rep copies of a head summed.  Reference :46-50."""
    if n_rep == 1:
        return grad_output
    return grad_output.unflatten(1, (grad_output.shape[1] // n_rep, n_rep)).sum(dim=2)


def unpad_input(hidden_states, attention_mask):
    """[B, S, ...] and a key-padding mask [B, S] (non-zero = a real token) -> (the real tokens' rows
    [nnz, ...], their positions in the flattened [B * S] axis, cumulative sequence lengths int32 [B + 1], the
    longest sequence as an int).  Reference :69-97 (flash-attn's padding helper; its map-free layers call it,
    the ones in this package mask instead).  Reads the longest length back from the device, as there."""
    lengths = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    cu_seqlens = torch.nn.functional.pad(torch.cumsum(lengths, dim=0, dtype=torch.int32), (1, 0))
    rows = hidden_states.reshape(-1, *hidden_states.shape[2:])
    return rows[indices], indices, cu_seqlens, int(lengths.max().item())


def pad_input(hidden_states, indices, batch, seqlen):
    """Inverse of unpad_input: rows [nnz, ...] back at `indices` of a zero-filled [batch, seqlen, ...].
    Reference :53-66."""
    out = hidden_states.new_zeros((batch * seqlen,) + tuple(hidden_states.shape[1:]))
    out[indices] = hidden_states
    return out.reshape(batch, seqlen, *hidden_states.shape[1:])


from ..operators.rope_kernels import rope_backward, rope_forward  # noqa: E402,F401  (in place, HIP)
