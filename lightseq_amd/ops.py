"""Torch-tensor wrappers of the operator launchers of the quantised layer path
(``include/lightseq_ops.h``; the reference's ``launch_*`` family of
lightseq/csrc/kernels/cuda/includes/kernels.h, bound there as ``torch_launch_*`` in
pybind/pybind_kernel_cuda.cpp).

Names and argument order follow the C++ launchers; the stream is torch's current stream and
the storage type is taken from the dtype of the T-typed tensors.  Clip values are device
tensors.  Mask tensors may be ``None``.  Dropout ratios must be 0.
"""
from .kernels import _dev, _suffix
from .lib import call, current_stream, ptr


def launch_quantize(q, clip_mask, alpha, f, clip_max, numel, mask_start_bit=2):
    _dev(q, clip_mask, alpha, f, clip_max)
    call("lsh_launch_quantize" + _suffix(f), ptr(q), ptr(clip_mask), ptr(alpha), ptr(f),
         ptr(clip_max), numel, mask_start_bit, current_stream())


def launch_quantize_2d(q, clip_mask, alpha, f, clip_max, batch_tokens, hidden_size,
                       mask_start_bit=2, out_layout=0):
    _dev(q, clip_mask, alpha, f, clip_max)
    call("lsh_launch_quantize_2d" + _suffix(f), ptr(q), ptr(clip_mask), ptr(alpha), ptr(f),
         ptr(clip_max), batch_tokens, hidden_size, mask_start_bit, current_stream(), out_layout)


def launch_fake_quantize(clip_mask, alpha, output, inp, clip_max, numel, mask_start_bit=2,
                         symmetry=True):
    _dev(clip_mask, alpha, output, inp, clip_max)
    call("lsh_launch_fake_quantize" + _suffix(inp), ptr(clip_mask), ptr(alpha), ptr(output),
         ptr(inp), ptr(clip_max), numel, mask_start_bit, current_stream(), int(symmetry))


def launch_dequantize(f, q, clip_max, numel, mask_start_bit=2):
    _dev(f, q, clip_max)
    call("lsh_launch_dequantize" + _suffix(f), ptr(f), ptr(q), ptr(clip_max), numel,
         mask_start_bit, current_stream())


def launch_layer_norm(ln_res, vars_, means, inp, scale, bias, batch_size, hidden_dim):
    _dev(ln_res, vars_, means, inp, scale, bias)
    call("lsh_launch_layer_norm" + _suffix(inp), ptr(ln_res), ptr(vars_), ptr(means), ptr(inp),
         ptr(scale), ptr(bias), batch_size, hidden_dim, current_stream())


def launch_layer_norm_i8(q_out, clip_mask_out, vars_, means, inp, gamma, betta, clip_max_out,
                         batch_size, hidden_dim):
    _dev(q_out, clip_mask_out, vars_, means, inp, gamma, betta, clip_max_out)
    call("lsh_launch_layer_norm_i8" + _suffix(inp), ptr(q_out), ptr(clip_mask_out), ptr(vars_),
         ptr(means), ptr(inp), ptr(gamma), ptr(betta), ptr(clip_max_out), batch_size, hidden_dim,
         current_stream())


def launch_attn_softmax(vals, attn_mask, batch_size, heads, from_len, to_len, mask_future=False):
    _dev(vals, attn_mask)
    call("lsh_launch_attn_softmax" + _suffix(vals), ptr(vals), ptr(attn_mask), batch_size, heads,
         from_len, to_len, int(mask_future), current_stream())


def launch_quant_bias_add_transform_20314(output, clip_mask, inp, bias, clip_max, dim_0, dim_1,
                                          dim_2, dim_3, dim_4, out_clip_max=None, in_col32=False):
    _dev(output, clip_mask, inp, bias, clip_max, out_clip_max)
    call("lsh_launch_quant_bias_add_transform_20314" + _suffix(output), ptr(output),
         ptr(clip_mask), ptr(inp), ptr(bias), ptr(clip_max), dim_0, dim_1, dim_2, dim_3, dim_4,
         current_stream(), ptr(out_clip_max), int(in_col32))


def launch_bias_add_transform_20314(output, inp, bias, dim_0, dim_1, dim_2, dim_3, dim_4):
    """kernels.h:72-75: [d0, d1, d2, d3, d4] + bias [d2, d3, d4] -> [d2, d0, d3, d1, d4]."""
    _dev(output, inp, bias)
    call("lsh_launch_bias_add_transform_20314" + _suffix(output), ptr(output), ptr(inp),
         ptr(bias), dim_0, dim_1, dim_2, dim_3, dim_4, current_stream())


def launch_concat3_dim1(inp1, inp2, output, sz0, sz2, sz1_1, sz1_2):
    """kernels.h:183-185: [sz0, sz1_1, sz2] ++ [sz0, sz1_2, sz2] along dimension 1."""
    _dev(inp1, inp2, output)
    call("lsh_launch_concat3_dim1" + _suffix(output), ptr(inp1), ptr(inp2), ptr(output), sz0,
         sz2, sz1_1, sz1_2, current_stream())


def launch_transform4d_0213(output, vals, batch_size, seq_len, hidden_dim, nhead, trans_count):
    _dev(output, vals)
    call("lsh_launch_transform4d_0213" + _suffix(vals), ptr(output), ptr(vals), batch_size,
         seq_len, hidden_dim, nhead, trans_count, current_stream())


def launch_quant_transform4d_0213(output, clip_mask, vals, clip_max, batch_size, seq_len,
                                  hidden_dim, nhead, trans_count):
    _dev(output, clip_mask, vals, clip_max)
    call("lsh_launch_quant_transform4d_0213" + _suffix(vals), ptr(output), ptr(clip_mask),
         ptr(vals), ptr(clip_max), batch_size, seq_len, hidden_dim, nhead, trans_count,
         current_stream())


def launch_ls_dropout(out, vals, mask, total_count, ratio=0.0, backward=False):
    _dev(out, vals, mask)
    call("lsh_launch_ls_dropout" + _suffix(vals), ptr(out), ptr(vals), ptr(mask), total_count,
         ratio, current_stream(), int(backward))


def launch_ls_dropout_res_bias(out, vals, mask, bias, residual, total_count, dim, ratio=0.0):
    _dev(out, vals, mask, bias, residual)
    call("lsh_launch_ls_dropout_res_bias" + _suffix(vals), ptr(out), ptr(vals), ptr(mask),
         ptr(bias), ptr(residual), total_count, dim, ratio, current_stream())


def launch_ls_dropout_act_bias(act, out, vals, mask, bias, total_count, dim, ratio=0.0):
    """``act``: "gelu" or "relu" (the template argument of the reference launcher)."""
    _dev(out, vals, mask, bias)
    call("lsh_launch_ls_dropout_act_bias_%s%s" % (act, _suffix(vals)), ptr(out), ptr(vals),
         ptr(mask), ptr(bias), total_count, dim, ratio, current_stream())


def launch_ls_quant_dropout_act_bias(act, qout, cmask_out, cmask_in, dropout_mask, qinput, bias,
                                     cmax_out, cmax_in, total_count, dim, ratio=0.0):
    _dev(qout, cmask_out, cmask_in, dropout_mask, qinput, bias, cmax_out, cmax_in)
    call("lsh_launch_ls_quant_dropout_act_bias_%s%s" % (act, _suffix(bias)), ptr(qout),
         ptr(cmask_out), ptr(cmask_in), ptr(dropout_mask), ptr(qinput), ptr(bias), ptr(cmax_out),
         ptr(cmax_in), total_count, dim, ratio, current_stream())


def launch_ls_fakequant_dropout_act_bias(act, out, cmask_out, cmask_in, dropout_mask, qinput,
                                         bias, cmax_out, cmax_in, total_count, dim, ratio=0.0,
                                         in_col32=False, symmetry=True):
    _dev(out, cmask_out, cmask_in, dropout_mask, qinput, bias, cmax_out, cmax_in)
    call("lsh_launch_ls_fakequant_dropout_act_bias_%s%s" % (act, _suffix(bias)), ptr(out),
         ptr(cmask_out), ptr(cmask_in), ptr(dropout_mask), ptr(qinput), ptr(bias), ptr(cmax_out),
         ptr(cmax_in), total_count, dim, ratio, current_stream(), int(in_col32), int(symmetry))


def launch_ls_quant_dropout_res_bias(out, mask, qvals, cmax, bias, residual, total_count, dim,
                                     ratio=0.0, in_col32=False):
    _dev(out, mask, qvals, cmax, bias, residual)
    call("lsh_launch_ls_quant_dropout_res_bias" + _suffix(out), ptr(out), ptr(mask), ptr(qvals),
         ptr(cmax), ptr(bias), ptr(residual), total_count, dim, ratio, current_stream(),
         int(in_col32))


def feed_forward_i8(bsz, output_size, input_size, qinput, qweight, alpha, beta, qout):
    """``FeedForward<T>::Forward`` int8 overload (ops/includes/feed_forward.h:46-79)."""
    _dev(qinput, qweight, alpha, beta, qout)
    call("lsh_feed_forward_i8", bsz, output_size, input_size, ptr(qinput), ptr(qweight),
         ptr(alpha), ptr(beta), ptr(qout), current_stream())


def strided_batch_gemm(bsz, m, n, k, alpha, beta, op_a, op_b, buffer_a, buffer_b, output):
    """``StridedBatchGemm<T>::Forward`` (ops/includes/strided_batch_gemm.h:45-57); op 0 = N,
    1 = T; column-major cuBLAS semantics with strides m*k, n*k, m*n."""
    _dev(buffer_a, buffer_b, output)
    call("lsh_strided_batch_gemm" + _suffix(output), bsz, m, n, k, float(alpha), float(beta),
         int(op_a), int(op_b), ptr(buffer_a), ptr(buffer_b), ptr(output), current_stream())


def layer_attention(q, k, v, attn_mask, ctx, batch_size, seq_len, heads, dim_per_head,
                    mask_future=False):
    _dev(q, k, v, attn_mask, ctx)
    call("lsh_layer_attention_f16", ptr(q), ptr(k), ptr(v), ptr(attn_mask), ptr(ctx), batch_size,
         seq_len, heads, dim_per_head, int(mask_future), current_stream())


def layer_cross_attention(q, k, v, attn_mask, ctx, batch_size, from_len, to_len, heads,
                          dim_per_head, mask_future=False):
    """Attention core with its own number of keys (cross attention, cached decoding step)."""
    _dev(q, k, v, attn_mask, ctx)
    call("lsh_layer_cross_attention_f16", ptr(q), ptr(k), ptr(v), ptr(attn_mask), ptr(ctx),
         batch_size, from_len, to_len, heads, dim_per_head, int(mask_future), current_stream())
