"""Launcher wrappers over the C ABI that take torch tensors.

Names, argument order and meaning follow the reference launchers
(lightseq/inference/kernels/transformerKernels_int8.h, embKernels_int8.h,
transformerKernels.h, model/cublas_helper.h); the stream is torch's current
stream, ``max_thread_per_block`` is accepted and ignored (the HIP kernels choose
their own launch shape) and COL32 flags must stay False.  The storage type T is
taken from the dtype of the T-typed tensors (float16 / float32).
"""
import torch

from . import lib
from .lib import call, current_stream, ptr


def _suffix(t):
    if t.dtype == torch.float16:
        return "_f16"
    if t.dtype == torch.float32:
        return "_f32"
    raise TypeError("T tensors must be float16 or float32, got %s" % t.dtype)


def _dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("all tensors must live on the GPU (no CPU fallback exists)")


def launch_quantize_tensor(inp, out, batch_tokens, hidden_size, quant_scale, out_col32=False):
    _dev(inp, out)
    call("lsh_launch_quantize_tensor" + _suffix(inp), ptr(inp), ptr(out), batch_tokens,
         hidden_size, quant_scale, current_stream(), int(out_col32))


def launch_dequantize_tensor(inp, out, batch_tokens, hidden_size, dequant_scale, in_col32=False):
    _dev(inp, out)
    call("lsh_launch_dequantize_tensor" + _suffix(out), ptr(inp), ptr(out), batch_tokens,
         hidden_size, dequant_scale, current_stream(), int(in_col32))


def ker_norm_layer_resual_i8O_launcher(token_num, hidden_size, inp, out, scale, bias,
                                       residual_bias, max_thread_per_block, quant_scale,
                                       is_post_ln=False, out_col32=False):
    _dev(inp, out, scale, bias, residual_bias)
    call("lsh_ker_norm_layer_resual_i8O" + _suffix(inp), token_num, hidden_size, current_stream(),
         ptr(inp), ptr(out), ptr(scale), ptr(bias), ptr(residual_bias), max_thread_per_block,
         quant_scale, int(is_post_ln), int(out_col32))


def ker_residual_bias_ln_i32I_i8O_launcher(inp, scale, bias, residual_bias, out, residual,
                                           batch_tokens, hidden_size, dequant_scale, quant_scale,
                                           max_thread_per_block, is_post_ln=False, in_col32=False,
                                           out_col32=False, colsum=None):
    _dev(inp, scale, bias, residual_bias, out, residual, colsum)
    call("lsh_ker_residual_bias_ln_i32I_i8O" + _suffix(residual), ptr(inp), ptr(scale), ptr(bias),
         ptr(residual_bias), ptr(out), ptr(residual), batch_tokens, hidden_size, dequant_scale,
         quant_scale, max_thread_per_block, current_stream(), int(is_post_ln), int(in_col32),
         int(out_col32), ptr(colsum))


def ker_residual_bias_ln_i8I_i8O_launcher(inp, scale, bias, residual_bias, out, residual,
                                          batch_tokens, hidden_size, dequant_scale, quant_scale,
                                          max_thread_per_block, is_post_ln=False, in_col32=False,
                                          out_col32=False, colsum=None):
    _dev(inp, scale, bias, residual_bias, out, residual, colsum)
    call("lsh_ker_residual_bias_ln_i8I_i8O" + _suffix(residual), ptr(inp), ptr(scale), ptr(bias),
         ptr(residual_bias), ptr(out), ptr(residual), batch_tokens, hidden_size, dequant_scale,
         quant_scale, max_thread_per_block, current_stream(), int(is_post_ln), int(in_col32),
         int(out_col32), ptr(colsum))


def ker_residual_bias_ln_i32I_launcher(inp, scale, bias, residual, out, batch_tokens, hidden_size,
                                       dequant_scale, max_thread_per_block, in_col32=False,
                                       colsum=None):
    _dev(inp, scale, bias, residual, out, colsum)
    call("lsh_ker_residual_bias_ln_i32I" + _suffix(residual), ptr(inp), ptr(scale), ptr(bias),
         ptr(residual), ptr(out), batch_tokens, hidden_size, dequant_scale, max_thread_per_block,
         current_stream(), int(in_col32), ptr(colsum))


def ker_bias_gelu_i8I_i8O_launcher(batch_token_num, inp, out, bias, feature_dim, dequant_scale,
                                   quant_scale, in_col32=False, out_col32=False):
    _dev(inp, out, bias)
    call("lsh_ker_bias_gelu_i8I_i8O" + _suffix(bias), batch_token_num, current_stream(), ptr(inp),
         ptr(out), ptr(bias), feature_dim, dequant_scale, quant_scale, int(in_col32),
         int(out_col32))


def ker_bias_relu_i8I_i8O_launcher(batch_token_num, inp, out, bias, feature_dim, dequant_scale,
                                   quant_scale, clip_max, in_col32=False, out_col32=False,
                                   narrow_clip=False):
    _dev(inp, out, bias)
    call("lsh_ker_bias_relu_i8I_i8O" + _suffix(bias), batch_token_num, current_stream(), ptr(inp),
         ptr(out), ptr(bias), feature_dim, dequant_scale, quant_scale, clip_max, int(in_col32),
         int(out_col32), int(narrow_clip))


def ker_arrange_encself_qkv_i8I_launcher(batch_token_num, hidden_size, ori_qkv, qkv_bias, new_qkv,
                                         max_batch_dim, batch_seq_len, dim_per_head, head_num,
                                         max_thread_per_block, dequant_scale, in_col32=False):
    _dev(ori_qkv, qkv_bias, new_qkv)
    call("lsh_ker_arrange_encself_qkv_i8I" + _suffix(new_qkv), batch_token_num, hidden_size,
         current_stream(), ptr(ori_qkv), ptr(qkv_bias), ptr(new_qkv), max_batch_dim, batch_seq_len,
         dim_per_head, head_num, max_thread_per_block, dequant_scale, int(in_col32))


def ker_arrange_encself_qkv_i8I_i8O_launcher(batch_token_num, hidden_size, ori_qkv, qkv_bias,
                                             new_q, new_k, new_v, d_v, batch_seq_len, dim_per_head,
                                             head_num, max_thread_per_block, dequant_scale,
                                             quant_scale, in_col32=False):
    _dev(ori_qkv, qkv_bias, new_q, new_k, new_v, d_v)
    call("lsh_ker_arrange_encself_qkv_i8I_i8O" + _suffix(d_v), batch_token_num, hidden_size,
         current_stream(), ptr(ori_qkv), ptr(qkv_bias), ptr(new_q), ptr(new_k), ptr(new_v),
         ptr(d_v), batch_seq_len, dim_per_head, head_num, max_thread_per_block, dequant_scale,
         quant_scale, int(in_col32))


def ker_arrange_atten_output_i8O_launcher(batch_token_num, hidden_size, ori_q, new_q, beam_size,
                                          dim_per_head, head_num, max_thread_per_block,
                                          quant_scale, out_col32=False):
    _dev(ori_q, new_q)
    call("lsh_ker_arrange_atten_output_i8O" + _suffix(ori_q), batch_token_num, hidden_size,
         current_stream(), ptr(ori_q), ptr(new_q), beam_size, dim_per_head, head_num,
         max_thread_per_block, quant_scale, int(out_col32))


def ker_correlation_softmax_encself_launcher(batch_size, batch_seq_len, head_num, correlation,
                                             src_padding_mask):
    _dev(correlation, src_padding_mask)
    call("lsh_ker_correlation_softmax_encself" + _suffix(correlation), batch_size, batch_seq_len,
         head_num, current_stream(), ptr(correlation), ptr(src_padding_mask))


def encself_attention(q, k, v, src_padding_mask, ctx, ctx_q, quant_scale, batch_size,
                      batch_seq_len, head_num, dim_per_head):
    """Fused scaled-dot-product attention of the encoder (fp16 only)."""
    _dev(q, k, v, src_padding_mask, ctx, ctx_q)
    if q.dtype != torch.float16:
        raise TypeError("encself_attention is fp16 only")
    call("lsh_encself_attention_f16", ptr(q), ptr(k), ptr(v), ptr(src_padding_mask), ptr(ctx),
         ptr(ctx_q), quant_scale, batch_size, batch_seq_len, head_num, dim_per_head,
         current_stream())


def launch_enc_emb_i8I(token_emb, pos_emb, tokens, output, pad_mask, pad_id, batch_size, seq_len,
                       hidden_dim, lang_emb, lang_id, multilg_type, dequant_scale, scaled):
    _dev(token_emb, pos_emb, tokens, output, pad_mask)
    call("lsh_launch_enc_emb_i8I" + _suffix(output), ptr(token_emb), ptr(pos_emb), ptr(tokens),
         ptr(output), ptr(pad_mask), pad_id, batch_size, seq_len, hidden_dim, current_stream(),
         ptr(lang_emb), ptr(lang_id), multilg_type, dequant_scale, int(scaled))


def launch_scaled_colsum(inp, out, rows, cols, scale):
    _dev(inp, out)
    call("lsh_launch_scaled_colsum" + _suffix(inp), ptr(inp), ptr(out), rows, cols, scale,
         current_stream())


def gemm_i8_i32o(a, w, c, m, n, k):
    """c[m,n] (int32) = a[m,k] @ w[n,k]^T."""
    _dev(a, w, c)
    call("lsh_gemm_i8_i32o", ptr(a), ptr(w), ptr(c), m, n, k, current_stream())


def gemm_i8_i8o(a, w, c, m, n, k, alpha):
    """c[m,n] (int8) = clamp(floor(alpha * (a @ w^T) + 0.5), -127, 127)."""
    _dev(a, w, c)
    call("lsh_gemm_i8_i8o", ptr(a), ptr(w), ptr(c), m, n, k, alpha, current_stream())


def gemm_i8_bias_gelu_i8o(a, w, c, bias, m, n, k, alpha, dequant_scale, quant_scale):
    """int8-output GEMM fused with ker_bias_gelu_i8I_i8O (fp16 bias)."""
    _dev(a, w, c, bias)
    call("lsh_gemm_i8_bias_gelu_i8o_f16", ptr(a), ptr(w), ptr(c), ptr(bias), m, n, k, alpha,
         dequant_scale, quant_scale, current_stream())


def gemm_i8_bias_relu_i8o(a, w, c, bias, m, n, k, alpha, dequant_scale, quant_scale, clip_max,
                          narrow_clip):
    """int8-output GEMM fused with ker_bias_relu_i8I_i8O (fp16 bias)."""
    _dev(a, w, c, bias)
    call("lsh_gemm_i8_bias_relu_i8o_f16", ptr(a), ptr(w), ptr(c), ptr(bias), m, n, k, alpha,
         dequant_scale, quant_scale, clip_max, int(narrow_clip), current_stream())


def gemm_i8_qkv_arrange(a, w, new_qkv, qkv_bias, max_batch_dim, batch_token_num, hidden_size, k,
                        batch_seq_len, head_num, alpha, dequant_scale):
    """QKV int8-output GEMM fused with ker_arrange_encself_qkv_i8I (fp16)."""
    _dev(a, w, new_qkv, qkv_bias)
    call("lsh_gemm_i8_qkv_arrange_f16", ptr(a), ptr(w), ptr(new_qkv), ptr(qkv_bias), max_batch_dim,
         batch_token_num, hidden_size, k, batch_seq_len, head_num, alpha, dequant_scale,
         current_stream())


def quantize_weight(host_weight, dev_q, rows, cols, quant_scale, layout):
    """``host_weight``: CPU tensor [rows, cols]; layout 0 = kRowMajor, 1 = kColMajor."""
    if host_weight.is_cuda:
        raise ValueError("quantize_weight takes a host tensor, as the reference does")
    _dev(dev_q)
    call("lsh_quantize_weight" + _suffix(host_weight), ptr(host_weight), ptr(dev_q), rows, cols,
         quant_scale, current_stream(), layout)


__all__ = [n for n in dir() if n.startswith(("launch_", "ker_", "gemm_", "encself_", "quantize_"))]
_ = lib  # re-exported for callers that want lib.LSHError
