"""Launcher wrappers over the C ABI that take torch tensors.

Names, argument order and meaning follow the reference launchers
(lightseq/inference/kernels/transformerKernels_int8.h, embKernels_int8.h,
transformerKernels.h, model/cublas_helper.h); the stream is torch's current
stream, ``max_thread_per_block`` is accepted and ignored (the HIP kernels choose
their own launch shape) and COL32 flags must stay False.  The storage type T is
taken from the dtype of the T-typed tensors (float16 / float32).
"""
import ctypes

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


def encself_attention_i8qkv(qkv, qkv_bias, dequant_scale, src_padding_mask, ctx, ctx_q, quant_scale,
                            batch_size, batch_seq_len, head_num, dim_per_head):
    """Fused encoder attention fed by the int8 output of the QKV product [tokens, 3 * hidden]
    and the fp16 bias [3 * hidden] (ker_arrange_encself_qkv_i8I applied while reading)."""
    _dev(qkv, qkv_bias, src_padding_mask, ctx, ctx_q)
    if qkv.dtype != torch.int8 or qkv_bias.dtype != torch.float16:
        raise TypeError("encself_attention_i8qkv takes int8 codes and an fp16 bias")
    call("lsh_encself_attention_i8qkv_f16", ptr(qkv), ptr(qkv_bias), dequant_scale,
         ptr(src_padding_mask), ptr(ctx), ptr(ctx_q), quant_scale, batch_size, batch_seq_len,
         head_num, dim_per_head, current_stream())


def qkv_attention_i8(x, qkv_weight, qkv_bias, src_padding_mask, ctx_q, requant_alpha, dequant_scale,
                     quant_scale, batch_size, batch_seq_len, head_num, dim_per_head):
    """QKV projection + encoder attention in one kernel (heads of 64, at most 128 tokens):
    the same bytes as gemm_i8_i8o(alpha=requant_alpha) followed by encself_attention_i8qkv."""
    _dev(x, qkv_weight, qkv_bias, src_padding_mask, ctx_q)
    if x.dtype != torch.int8 or qkv_weight.dtype != torch.int8 or qkv_bias.dtype != torch.float16:
        raise TypeError("qkv_attention_i8 takes int8 activations and weights and an fp16 bias")
    call("lsh_qkv_attention_i8_f16", ptr(x), ptr(qkv_weight), ptr(qkv_bias), ptr(src_padding_mask),
         ptr(ctx_q), requant_alpha, dequant_scale, quant_scale, batch_size, batch_seq_len, head_num,
         dim_per_head, current_stream())


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


def gemm_i8_i32o_splitk(a, w, c, m, n, k, ksplit):
    """K split into ``ksplit`` ranges; range p fills the plane c[p] of c [ksplit, m, n].
    Returns the split applied."""
    import ctypes
    _dev(a, w, c)
    used = ctypes.c_int(0)
    call("lsh_gemm_i8_i32o_splitk", ptr(a), ptr(w), ptr(c), m, n, k, ksplit,
         ctypes.cast(ctypes.byref(used), ctypes.c_void_p), current_stream())
    return used.value


def layer_norm_row_kernel(on):
    """Select (True) or deselect the workgroup-per-row layer-norm kernel for this thread's
    later launches; returns the previous setting."""
    return bool(lib.load().lsh_layer_norm_row_kernel(int(bool(on))))


def gemm_i8_preferred_ksplit(m, n, k):
    return lib.load().lsh_gemm_i8_preferred_ksplit(m, n, k)


def ker_residual_bias_ln_planes_i32I_i8O(inp, nparts, part_stride, scale, bias, residual_bias, out,
                                         residual, batch_tokens, hidden_size, dequant_scale,
                                         quant_scale, is_post_ln=False, colsum=None):
    _dev(inp, scale, bias, residual_bias, out, residual, colsum)
    call("lsh_ker_residual_bias_ln_planes_i32I_i8O_f16", ptr(inp), nparts, part_stride, ptr(scale),
         ptr(bias), ptr(residual_bias), ptr(out), ptr(residual), batch_tokens, hidden_size,
         dequant_scale, quant_scale, current_stream(), int(is_post_ln), ptr(colsum))


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


# --------------------------------------------------------------------------- #
# decoder step
# --------------------------------------------------------------------------- #
def launch_dec_emb_i8I(token_emb, pos_emb, tokens, lang_emb, lang_id, output, batch_size,
                       beam_size, hidden_dim, vocab_size, step, max_step, multilg_type,
                       dequant_scale, scaled, vocab_major=False):
    """``vocab_major``: ``token_emb`` is [vocab, hidden] instead of the reference's
    [hidden, vocab]."""
    _dev(token_emb, pos_emb, tokens, output)
    name = "lsh_launch_dec_emb_i8I_vocab_major" if vocab_major else "lsh_launch_dec_emb_i8I"
    call(name + _suffix(output), ptr(token_emb), ptr(pos_emb), ptr(tokens), ptr(lang_emb),
         ptr(lang_id), ptr(output), batch_size, beam_size, hidden_dim, vocab_size, step, max_step,
         multilg_type, current_stream(), dequant_scale, int(scaled))


def ker_arrange_decself_qkv_i8I_i8O_launcher(step_token_num, hidden_size, ori_qkv, qkv_bias, new_q,
                                             new_k, new_v, head_num, dim_per_head, max_step,
                                             step_id, max_thread_per_block, dequant_scale,
                                             quant_scale, in_col32=False):
    _dev(ori_qkv, qkv_bias, new_q, new_k, new_v)
    call("lsh_ker_arrange_decself_qkv_i8I_i8O" + _suffix(qkv_bias), step_token_num, hidden_size,
         current_stream(), ptr(ori_qkv), ptr(qkv_bias), ptr(new_q), ptr(new_k), ptr(new_v),
         head_num, dim_per_head, max_step, step_id, max_thread_per_block, dequant_scale,
         quant_scale, int(in_col32))


def decself_scores_i8_i32o(k_cache, q, scores, batch_head_num, step_num, max_step, dim_per_head):
    _dev(k_cache, q, scores)
    call("lsh_decself_scores_i8_i32o", ptr(k_cache), ptr(q), ptr(scores), batch_head_num, step_num,
         max_step, dim_per_head, current_stream())


def ker_fuse_softmax_new_value_i32I_i8O_launcher(correlation, v, new_v, batch_head_num, step_num,
                                                 max_step, head_num, dim_per_head, attn_scale,
                                                 dequant_scale, quant_scale, out_col32=False):
    _dev(correlation, v, new_v)
    call("lsh_ker_fuse_softmax_new_value_i32I_i8O", ptr(correlation), ptr(v), ptr(new_v),
         batch_head_num, step_num, max_step, head_num, dim_per_head, attn_scale, dequant_scale,
         quant_scale, int(out_col32), current_stream())


def decself_attention_i8(q, k_cache, v_cache, new_v, batch_head_num, step_num, max_step, head_num,
                         dim_per_head, attn_scale, dequant_scale, quant_scale):
    """Scores + softmax + new value of the decoder self attention in one kernel."""
    _dev(q, k_cache, v_cache, new_v)
    call("lsh_decself_attention_i8", ptr(q), ptr(k_cache), ptr(v_cache), ptr(new_v),
         batch_head_num, step_num, max_step, head_num, dim_per_head, attn_scale, dequant_scale,
         quant_scale, current_stream())


def ker_arrange_encdec_q_i8I_launcher(step_token_num, hidden_size, ori_q, q_bias, new_q, beam_size,
                                      dim_per_head, head_num, max_thread_per_block, dequant_scale,
                                      in_col32=False):
    _dev(ori_q, q_bias, new_q)
    call("lsh_ker_arrange_encdec_q_i8I" + _suffix(new_q), step_token_num, hidden_size,
         current_stream(), ptr(ori_q), ptr(q_bias), ptr(new_q), beam_size, dim_per_head, head_num,
         max_thread_per_block, dequant_scale, int(in_col32))


def ker_arrange_encdec_kv_launcher(batch_token_num, dec_layer_num, hidden_size, ori_kv, kv_bias,
                                   new_k, new_v, offset_per_layer, batch_seq_len, dim_per_head,
                                   head_num, max_thread_per_block):
    _dev(ori_kv, kv_bias, new_k, new_v)
    call("lsh_ker_arrange_encdec_kv" + _suffix(ori_kv), batch_token_num, dec_layer_num,
         hidden_size, current_stream(), ptr(ori_kv), ptr(kv_bias), ptr(new_k), ptr(new_v),
         offset_per_layer, batch_seq_len, dim_per_head, head_num, max_thread_per_block)


def ker_correlation_softmax_encdec_launcher(batch_size, head_num_per_seq, batch_seq_len,
                                            correlation, src_padding_mask):
    _dev(correlation, src_padding_mask)
    call("lsh_ker_correlation_softmax_encdec" + _suffix(correlation), batch_size, head_num_per_seq,
         batch_seq_len, current_stream(), ptr(correlation), ptr(src_padding_mask))


def encdec_attention(q, k, v, pad_mask, ctx, ctx_q, quant_scale, batch_size, beam_size, head_num,
                     batch_seq_len, dim_per_head):
    """Fused encoder-decoder attention of one decoder layer (fp16 only)."""
    _dev(q, k, v, pad_mask, ctx, ctx_q)
    if q.dtype != torch.float16:
        raise TypeError("encdec_attention is fp16 only")
    call("lsh_encdec_attention_f16", ptr(q), ptr(k), ptr(v), ptr(pad_mask), ptr(ctx), ptr(ctx_q),
         quant_scale, batch_size, beam_size, head_num, batch_seq_len, dim_per_head,
         current_stream())


def gemm_f16_nt(a, w, c, m, n, k):
    """c[m,n] (fp16) = a[m,k] @ w[n,k]^T with fp32 accumulation."""
    _dev(a, w, c)
    call("lsh_gemm_f16_nt", ptr(a), ptr(w), ptr(c), m, n, k, current_stream())


# --------------------------------------------------------------------------- #
# beam search
# --------------------------------------------------------------------------- #
def length_norm(length, alpha):
    return lib.load().lsh_length_norm(int(length), float(alpha))


def select_beam_rough_topk_i8I_launcher(logits, logit_bias, seq_probs, seq_score, alive_seq,
                                        dequant_scale, can_idx, can_score, num_beam_can,
                                        vocab_size, max_step, length_norm_value, cur_step,
                                        step_token_num, max_thread_per_block, beam_size,
                                        diverse_lambda, end_id, in_col32=False):
    _dev(logits, logit_bias, seq_probs, seq_score, alive_seq, can_idx, can_score, num_beam_can)
    call("lsh_select_beam_rough_topk_i8I" + _suffix(logit_bias), ptr(logits), ptr(logit_bias),
         ptr(seq_probs), ptr(seq_score), ptr(alive_seq), dequant_scale, ptr(can_idx),
         ptr(can_score), ptr(num_beam_can), vocab_size, max_step, length_norm_value, cur_step,
         step_token_num, max_thread_per_block, current_stream(), beam_size, diverse_lambda, end_id,
         int(in_col32))


def ker_refresh_result(can_idx, can_score, num_can_per_beam, old_alive_seq, new_alive_seq,
                       seq_probs, seq_score, num_finish_beam, vocab_size, cur_step,
                       length_norm_value, diverse_lambda, end_id, batch_size, beam_size, max_step):
    """``num_can_per_beam`` may be an int (device address) to pass ``can_num + 1``."""
    _dev(can_idx, can_score, old_alive_seq, new_alive_seq, seq_probs, seq_score, num_finish_beam)
    ncp = num_can_per_beam if isinstance(num_can_per_beam, int) else ptr(num_can_per_beam)
    call("lsh_ker_refresh_result", ptr(can_idx), ptr(can_score), ncp, ptr(old_alive_seq),
         ptr(new_alive_seq), ptr(seq_probs), ptr(seq_score), ptr(num_finish_beam), vocab_size,
         cur_step, length_norm_value, diverse_lambda, end_id, batch_size, beam_size, max_step,
         current_stream())


def ker_refresh_cache_launcher_i8(grid_dim_x, grid_dim_y, block_dim, num_can_per_beam, can_idx,
                                  self_k_bgeem, self_v_bgeem, new_self_k_bgeem, new_self_v_bgeem,
                                  self_k_bgeem_offset, beam_size, dim_per_head, head_num,
                                  vocab_size, cur_step, max_step, diverse, end_id):
    _dev(can_idx, self_k_bgeem, self_v_bgeem, new_self_k_bgeem, new_self_v_bgeem)
    ncp = num_can_per_beam if isinstance(num_can_per_beam, int) else ptr(num_can_per_beam)
    call("lsh_ker_refresh_cache_i8", grid_dim_x, grid_dim_y, block_dim, current_stream(), ncp,
         ptr(can_idx), ptr(self_k_bgeem), ptr(self_v_bgeem), ptr(new_self_k_bgeem),
         ptr(new_self_v_bgeem), self_k_bgeem_offset, beam_size, dim_per_head, head_num, vocab_size,
         cur_step, max_step, int(diverse), end_id)


def ker_write_trg_tokenid_pos_penalty(alive_seq, seq_score, output, max_step, beam_size,
                                      batch_size, out_len):
    _dev(alive_seq, seq_score, output)
    call("lsh_ker_write_trg_tokenid_pos_penalty", ptr(alive_seq), ptr(seq_score), ptr(output),
         max_step, beam_size, batch_size, out_len, current_stream())


def ker_write_trg_tokenid_neg_penalty(alive_seq, seq_score, output, max_step, beam_size,
                                      vocab_size, end_id, batch_size, out_len):
    _dev(alive_seq, seq_score, output)
    call("lsh_ker_write_trg_tokenid_neg_penalty", ptr(alive_seq), ptr(seq_score), ptr(output),
         max_step, beam_size, vocab_size, end_id, batch_size, out_len, current_stream())


def ker_write_topk_result(alive_seq, seq_score, res_seq, vocab_size, max_step, beam_size, end_id,
                          batch_beam_num, out_len):
    _dev(alive_seq, seq_score, res_seq)
    call("lsh_ker_write_topk_result", ptr(alive_seq), ptr(seq_score), ptr(res_seq), vocab_size,
         max_step, beam_size, end_id, batch_beam_num, out_len, current_stream())


def beam_search_step_i8I(logits, logit_bias, seq_probs, seq_score, old_alive_seq, new_alive_seq,
                         top_score, top_idx, parent, num_finished, dequant_scale, vocab_size,
                         max_step, length_norm_value, cur_step, batch_size, beam_size, end_id):
    """Exact top-k per row + per-sentence merge + result refresh, all on the device."""
    _dev(logits, logit_bias, seq_probs, seq_score, old_alive_seq, new_alive_seq, top_score,
         top_idx, parent, num_finished)
    call("lsh_beam_search_step_i8I" + _suffix(logit_bias), ptr(logits), ptr(logit_bias),
         ptr(seq_probs), ptr(seq_score), ptr(old_alive_seq), ptr(new_alive_seq), ptr(top_score),
         ptr(top_idx), ptr(parent), ptr(num_finished), dequant_scale, vocab_size, max_step,
         length_norm_value, cur_step, batch_size, beam_size, end_id, current_stream())


def beam_search_step_workspace(batch_size, beam_size, vocab_size):
    """Bytes of the optional second workspace of :func:`beam_search_step_ws_i8I` (0: unused)."""
    f = lib.load().lsh_beam_search_step_workspace
    f.restype = ctypes.c_int64
    return int(f(int(batch_size), int(beam_size), int(vocab_size)))


def beam_search_step_ws_i8I(logits, logit_bias, seq_probs, seq_score, old_alive_seq, new_alive_seq,
                            top_score, top_idx, parent, num_finished, dequant_scale, vocab_size,
                            max_step, length_norm_value, cur_step, batch_size, beam_size, end_id,
                            workspace):
    """:func:`beam_search_step_i8I` with the per-row top-k dealt to several workgroups per row
    (``workspace``: a tensor of :func:`beam_search_step_workspace` bytes, or None)."""
    _dev(logits, logit_bias, seq_probs, seq_score, old_alive_seq, new_alive_seq, top_score,
         top_idx, parent, num_finished, workspace)
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    call("lsh_beam_search_step_ws_i8I" + _suffix(logit_bias), ptr(logits), ptr(logit_bias),
         ptr(seq_probs), ptr(seq_score), ptr(old_alive_seq), ptr(new_alive_seq), ptr(top_score),
         ptr(top_idx), ptr(parent), ptr(num_finished), dequant_scale, vocab_size, max_step,
         length_norm_value, cur_step, batch_size, beam_size, end_id, ptr(workspace), nbytes,
         current_stream())


def beam_search_step_noalloc_i8I(logits, logit_bias, seq_probs, seq_score, old_alive_seq,
                                 new_alive_seq, parent, num_finished, dequant_scale, vocab_size,
                                 max_step, length_norm_value, cur_step, batch_size, beam_size,
                                 end_id):
    """``beam_search_step_i8I`` (fp16 bias) with the proposal workspace inside the library:
    allocates nothing; batch_size * beam_size**2 <= 65536."""
    _dev(logits, logit_bias, seq_probs, seq_score, old_alive_seq, new_alive_seq, parent,
         num_finished)
    call("lsh_beam_search_step_noalloc_i8I_f16", ptr(logits), ptr(logit_bias), ptr(seq_probs),
         ptr(seq_score), ptr(old_alive_seq), ptr(new_alive_seq), ptr(parent), ptr(num_finished),
         dequant_scale, vocab_size, max_step, length_norm_value, cur_step, batch_size, beam_size,
         end_id, current_stream())


def refresh_cache_by_parent_i8(n_layer, rows, parent, k_old, v_old, k_new, v_new, layer_offset,
                               beam_size, dim_per_head, head_num, cur_step, max_step):
    _dev(parent, k_old, v_old, k_new, v_new)
    call("lsh_refresh_cache_by_parent_i8", n_layer, rows, current_stream(), ptr(parent),
         ptr(k_old), ptr(v_old), ptr(k_new), ptr(v_new), layer_offset, beam_size, dim_per_head,
         head_num, cur_step, max_step)


# --------------------------------------------------------------------------- #
# GPT path
# --------------------------------------------------------------------------- #
def ker_gpt_embedding_i8I_launcher(batch_size, batch_seq_len, hidden_size, token_emb, pos_emb,
                                   token_id, output, real_seq_len, padding_id, pos_offset,
                                   dequant_scale):
    _dev(token_emb, pos_emb, token_id, output, real_seq_len)
    call("lsh_ker_gpt_embedding_i8I" + _suffix(output), batch_size, batch_seq_len, hidden_size,
         current_stream(), ptr(token_emb), ptr(pos_emb), ptr(token_id), ptr(output),
         ptr(real_seq_len), padding_id, pos_offset, dequant_scale)


def gpt_scores_i8_i32o(k, q, scores, batch_head_num, batch_seq_len, dim_per_head):
    _dev(k, q, scores)
    call("lsh_gpt_scores_i8_i32o", ptr(k), ptr(q), ptr(scores), batch_head_num, batch_seq_len,
         dim_per_head, current_stream())


def ker_correlation_softmax_gpt_i32I_launcher(batch_size, batch_seq_len, head_num, correlation,
                                              output, real_seq_len, attn_scale, dequant_scale):
    _dev(correlation, output, real_seq_len)
    call("lsh_ker_correlation_softmax_gpt_i32I" + _suffix(output), batch_size, batch_seq_len,
         head_num, current_stream(), ptr(correlation), ptr(output), ptr(real_seq_len), attn_scale,
         dequant_scale)


def ker_arrange_qkv_with_cache_i8I_i8O_launcher(batch_token_num, hidden_size, ori_qkv, qkv_bias,
                                                new_q, new_k, k_cache, new_v, v_cache,
                                                batch_seq_len, dim_per_head, head_num,
                                                dequant_scale, quant_scale, in_col32=False):
    _dev(ori_qkv, qkv_bias, new_q, new_k, k_cache, new_v, v_cache)
    call("lsh_ker_arrange_qkv_with_cache_i8I_i8O" + _suffix(qkv_bias), batch_token_num,
         hidden_size, current_stream(), ptr(ori_qkv), ptr(qkv_bias), ptr(new_q), ptr(new_k),
         ptr(k_cache), ptr(new_v), ptr(v_cache), batch_seq_len, dim_per_head, head_num,
         dequant_scale, quant_scale, int(in_col32))


def ker_topk_sample_i8I_launcher(batch_size, batch_seq_len, logits_seq_len, max_thread_per_block,
                                 logits, old_input_ids, new_input_ids, real_seq_len, vocab_size, k,
                                 unfinished, curandstate, eos_id, dequant_scale, in_col32=False):
    _dev(logits, old_input_ids, new_input_ids, unfinished)
    call("lsh_ker_topk_sample_i8I", batch_size, batch_seq_len, logits_seq_len,
         max_thread_per_block, current_stream(), ptr(logits), ptr(old_input_ids),
         ptr(new_input_ids), ptr(real_seq_len), vocab_size, k, ptr(unfinished), ptr(curandstate),
         eos_id, dequant_scale, int(in_col32))


def ker_topp_sample_i8I_launcher(batch_size, batch_seq_len, logits_seq_len, max_thread_per_block,
                                 logits, old_input_ids, new_input_ids, real_seq_len, vocab_size, p,
                                 unfinished, curandstate, eos_id, dequant_scale, in_col32=False):
    _dev(logits, old_input_ids, new_input_ids, unfinished, curandstate)
    call("lsh_ker_topp_sample_i8I", batch_size, batch_seq_len, logits_seq_len,
         max_thread_per_block, current_stream(), ptr(logits), ptr(old_input_ids),
         ptr(new_input_ids), ptr(real_seq_len), vocab_size, p, ptr(unfinished), ptr(curandstate),
         eos_id, dequant_scale, int(in_col32))


def ker_topk_sample_i8I_dec_launcher(batch_size, batch_seq_len, max_step, logits_seq_len,
                                     max_thread_per_block, logits, logit_bias, old_input_ids,
                                     new_input_ids, vocab_size, k, all_finished, curandstate,
                                     eos_id, dequant_scale, in_col32=False):
    """Encoder-decoder ``ker_topk_sample_i8I_launcher`` (transformerKernels_int8.h:123-132): ids in
    place in ``old_input_ids`` [batch, max_step]; ``curandstate`` may be None for k == 1."""
    _dev(logits, logit_bias, old_input_ids, all_finished)
    call("lsh_ker_topk_sample_i8I_dec" + _suffix(logit_bias), batch_size, batch_seq_len, max_step,
         logits_seq_len, max_thread_per_block, current_stream(), ptr(logits), ptr(logit_bias),
         ptr(old_input_ids), ptr(new_input_ids), vocab_size, k, ptr(all_finished),
         ptr(curandstate), eos_id, dequant_scale, int(in_col32))


def ker_topp_sample_i8I_dec_launcher(batch_size, batch_seq_len, max_step, logits_seq_len,
                                     max_thread_per_block, logits, logit_bias, old_input_ids,
                                     new_input_ids, vocab_size, p, unfinished, curandstate, eos_id,
                                     dequant_scale, in_col32=False):
    """Encoder-decoder ``ker_topp_sample_i8I_launcher`` (transformerKernels_int8.h:134-143)."""
    _dev(logits, logit_bias, old_input_ids, unfinished, curandstate)
    call("lsh_ker_topp_sample_i8I_dec" + _suffix(logit_bias), batch_size, batch_seq_len, max_step,
         logits_seq_len, max_thread_per_block, current_stream(), ptr(logits), ptr(logit_bias),
         ptr(old_input_ids), ptr(new_input_ids), vocab_size, p, ptr(unfinished), ptr(curandstate),
         eos_id, dequant_scale, int(in_col32))


def ker_attention_mask_weights_i32I_launcher(batch_size, dst_seq_len, src_seq_len, head_num,
                                             correlation, output, real_seq_len, attn_scale,
                                             dequant_scale):
    """``ker_attention_mask_weights_i32I_launcher`` (gptKernels_int8.h:57-61)."""
    _dev(correlation, output, real_seq_len)
    call("lsh_ker_attention_mask_weights_i32I" + _suffix(output), batch_size, dst_seq_len,
         src_seq_len, head_num, current_stream(), ptr(correlation), ptr(output), ptr(real_seq_len),
         attn_scale, dequant_scale)


def rng_setup(batch_size, seed, device="cuda"):
    """Generator states of ``batch_size`` sequences for the random-sampling launchers (in place
    of the reference's curandState array): an int64 tensor [batch_size, 2] holding
    ``lsh_rng_state_t`` records {seed, sequence, draws}."""
    state = torch.zeros((batch_size, 2), dtype=torch.int64, device=device)
    call("lsh_rng_setup", ptr(state), batch_size, int(seed) & 0xFFFFFFFFFFFFFFFF, current_stream())
    return state


def ker_ppl_i8I_launcher(batch_size, batch_seq_len, max_thread_per_block, logits, input_ids,
                         real_seq_len, ppl, vocab_size, dequant_scale, in_col32=False):
    _dev(logits, input_ids, real_seq_len, ppl)
    call("lsh_ker_ppl_i8I", batch_size, batch_seq_len, max_thread_per_block, current_stream(),
         ptr(logits), ptr(input_ids), ptr(real_seq_len), ptr(ppl), vocab_size, dequant_scale,
         int(in_col32))


def ker_ppl_i8I_workspace(batch_size, batch_seq_len, logits, input_ids, real_seq_len, ppl,
                          vocab_size, dequant_scale, workspace):
    """ker_ppl_i8I with one workgroup per position; workspace: batch * seq_len float32."""
    _dev(logits, input_ids, real_seq_len, ppl, workspace)
    if workspace.dtype != torch.float32 or workspace.numel() < batch_size * batch_seq_len:
        raise ValueError("workspace must hold batch_size * batch_seq_len float32")
    call("lsh_ker_ppl_i8I_workspace", batch_size, batch_seq_len, current_stream(), ptr(logits),
         ptr(input_ids), ptr(real_seq_len), ptr(ppl), vocab_size, dequant_scale, ptr(workspace))


def gpt_arrange_qkv_prefill(batch_token_num, hidden_size, ori_qkv, qkv_bias, q_codes, k_codes,
                            v_deq, k_cache, v_cache, batch_seq_len, dim_per_head, head_num,
                            max_step, dequant_scale, quant_scale):
    _dev(ori_qkv, qkv_bias, q_codes, k_codes, v_deq, k_cache, v_cache)
    call("lsh_gpt_arrange_qkv_prefill_f16", batch_token_num, hidden_size, current_stream(),
         ptr(ori_qkv), ptr(qkv_bias), ptr(q_codes), ptr(k_codes), ptr(v_deq), ptr(k_cache),
         ptr(v_cache), batch_seq_len, dim_per_head, head_num, max_step, dequant_scale, quant_scale)


def gpt_prefill_attention(q_codes, k_codes, v, real_seq_len, ctx, ctx_q, quant_scale,
                          dequant_scale, batch_size, batch_seq_len, head_num, dim_per_head):
    """Causal prompt attention of the int8 GPT path in one kernel (fp16 storage)."""
    _dev(q_codes, k_codes, v, real_seq_len, ctx, ctx_q)
    call("lsh_gpt_prefill_attention_f16", ptr(q_codes), ptr(k_codes), ptr(v), ptr(real_seq_len),
         ptr(ctx), ptr(ctx_q), quant_scale, dequant_scale, batch_size, batch_seq_len, head_num,
         dim_per_head, current_stream())


def gpt_prefill_i8_supported(batch_seq_len, head_num, dim_per_head):
    return bool(lib.load().lsh_gpt_prefill_i8_supported(int(batch_seq_len), int(head_num),
                                                        int(dim_per_head)))


def gpt_prefill_on_codes_in_models(on):
    """Switch QuantGpt's prompt pass between the int8-code kernels (default) and the fp16-storage
    pair; returns the previous setting."""
    return bool(lib.load().lsh_gpt_prefill_on_codes_in_models(int(bool(on))))


def gpt_arrange_qkv_prefill_i8(batch_token_num, hidden_size, ori_qkv, qkv_bias, q_codes, k_cache,
                               v_cache, batch_seq_len, dim_per_head, head_num, max_step,
                               dequant_scale, quant_scale):
    """ker_arrange_encself_qkv_i8I_i8O of the prompt pass with int8 outputs only: q codes
    [batch, head, seq, d], k / v codes into the caches [batch, head, max_step, d]."""
    _dev(ori_qkv, qkv_bias, q_codes, k_cache, v_cache)
    call("lsh_gpt_arrange_qkv_prefill_i8", batch_token_num, hidden_size, current_stream(),
         ptr(ori_qkv), ptr(qkv_bias), ptr(q_codes), ptr(k_cache), ptr(v_cache), batch_seq_len,
         dim_per_head, head_num, max_step, dequant_scale, quant_scale)


def gpt_prefill_attention_i8(q_codes, k_cache, v_cache, real_seq_len, ctx_q, quant_scale,
                             dequant_scale, v_quant_scale, batch_size, batch_seq_len, head_num,
                             dim_per_head, max_step):
    """Causal prompt attention of the int8 GPT path on the q codes and the caches."""
    _dev(q_codes, k_cache, v_cache, real_seq_len, ctx_q)
    call("lsh_gpt_prefill_attention_i8", ptr(q_codes), ptr(k_cache), ptr(v_cache),
         ptr(real_seq_len), ptr(ctx_q), quant_scale, dequant_scale, v_quant_scale, batch_size,
         batch_seq_len, head_num, dim_per_head, max_step, current_stream())


def gpt_greedy_step(logits, ids, last_ids, vocab_size, max_step, cur_len, batch_size, unfinished,
                    eos_id):
    _dev(logits, ids, last_ids, unfinished)
    call("lsh_gpt_greedy_step", ptr(logits), ptr(ids), ptr(last_ids), vocab_size, max_step,
         cur_len, batch_size, ptr(unfinished), eos_id, current_stream())


def gpt_sample_step(logits, ids, last_ids, vocab_size, max_step, cur_len, batch_size, unfinished,
                    eos_id, k, p, dequant_scale, state):
    """The model's step with random sampling: top-k for k in {2, 4, 8, 16, 32}, top-p for k == 0."""
    _dev(logits, ids, last_ids, unfinished, state)
    call("lsh_gpt_sample_step", ptr(logits), ptr(ids), ptr(last_ids), vocab_size, max_step,
         cur_len, batch_size, ptr(unfinished), eos_id, k, p, dequant_scale, ptr(state),
         current_stream())


__all__ = [n for n in dir() if n.startswith(("launch_", "ker_", "gemm_", "rng_", "encself_", "quantize_", "gpt_",
                                             "decself_", "encdec_", "select_beam_", "beam_",
                                             "refresh_", "length_norm"))]
_ = lib  # re-exported for callers that want lib.LSHError


def build_act_lut(lut, bias, n, dequant_scale, quant_scale, clip_max, act):
    """lut [n, 256] int8: bias + activation + requantisation per (column, code); act 0 GELU,
    1 ReLU, 2 ReLU with the narrow unsigned clip."""
    _dev(lut, bias)
    call("lsh_build_act_lut", ptr(lut), ptr(bias), n, dequant_scale, quant_scale, clip_max, act,
         current_stream())


def gemm_i8_decself_qkv_i8o(a, w, qkv_bias, new_q, new_k, new_v, step_token_num, hidden, k, head_num,
                            max_step, step_id, alpha, dequant_scale, quant_scale):
    """Decode-step QKV product with ker_arrange_decself_qkv_i8I_i8O as its epilogue."""
    _dev(a, w, qkv_bias, new_q, new_k, new_v)
    call("lsh_gemm_i8_decself_qkv_i8o_f16", ptr(a), ptr(w), ptr(qkv_bias), ptr(new_q), ptr(new_k),
         ptr(new_v), step_token_num, hidden, k, head_num, max_step, step_id, alpha, dequant_scale,
         quant_scale, current_stream())


def qkv_attention_plan(src_padding_mask, batch, seq_len, head_num):
    """The plan of ``qkv_attention_i8`` launches with this padding mask: an int32 tensor
    [batch * head_num]."""
    _dev(src_padding_mask)
    plan = torch.zeros(batch * head_num, dtype=torch.int32, device=src_padding_mask.device)
    call("lsh_qkv_attention_plan", ptr(src_padding_mask), ptr(plan), batch, seq_len, head_num,
         current_stream())
    return plan


def qkv_attention_plan_in_models(on):
    """Let the encoder models plan their fused QKV + attention launches from the padding mask
    (default) or not; returns the previous setting."""
    return bool(lib.load().lsh_qkv_attention_plan_in_models(int(bool(on))))


def qkv_attention_planned_i8(x, qkv_weight, qkv_bias, src_padding_mask, plan, ctx_q, requant_alpha,
                             dequant_scale, quant_scale, batch, seq_len, head_num, dim_per_head):
    """``qkv_attention_i8`` that skips the blocks of padding and takes the pairs in the plan's order."""
    _dev(x, qkv_weight, qkv_bias, src_padding_mask, plan, ctx_q)
    call("lsh_qkv_attention_planned_i8_f16", ptr(x), ptr(qkv_weight), ptr(qkv_bias),
         ptr(src_padding_mask), ptr(plan), ptr(ctx_q), requant_alpha, dequant_scale, quant_scale,
         batch, seq_len, head_num, dim_per_head, current_stream())


def decself_qkv_attention_i8(x, w, qkv_bias, new_q, k_cache, v_cache, ctx, rows, hidden, head_num,
                             max_step, step_id, alpha, dequant_scale, cache_quant_scale, attn_scale,
                             cache_dequant_scale, ctx_quant_scale):
    """Decode-step QKV product, cache append and self attention of heads of 64 in one launch."""
    _dev(x, w, qkv_bias, new_q, k_cache, v_cache, ctx)
    call("lsh_decself_qkv_attention_i8_f16", ptr(x), ptr(w), ptr(qkv_bias), ptr(new_q), ptr(k_cache),
         ptr(v_cache), ptr(ctx), rows, hidden, head_num, max_step, step_id, alpha, dequant_scale,
         cache_quant_scale, attn_scale, cache_dequant_scale, ctx_quant_scale, current_stream())


def gemm_i8_encdec_q(a, w, q_bias, new_q, step_token_num, hidden, k, beam_size, head_num, alpha,
                     dequant_scale):
    """Decode-step cross-attention query product with ker_arrange_encdec_q_i8I as its epilogue."""
    _dev(a, w, q_bias, new_q)
    call("lsh_gemm_i8_encdec_q_f16", ptr(a), ptr(w), ptr(q_bias), ptr(new_q), step_token_num, hidden,
         k, beam_size, head_num, alpha, dequant_scale, current_stream())


def encdec_q_attention(x, q_weight, q_bias, k, v, pad_mask, ctx_q, quant_scale, batch_size, beam_size,
                       head_num, batch_seq_len, hidden, alpha, dequant_scale):
    """Decode step: cross-attention query product and the attention itself in one launch (heads
    of 64, short sources); the bytes of gemm_i8_encdec_q + encdec_attention."""
    _dev(x, q_weight, q_bias, k, v, pad_mask, ctx_q)
    call("lsh_encdec_q_attention_f16", ptr(x), ptr(q_weight), ptr(q_bias), ptr(k), ptr(v),
         ptr(pad_mask), ptr(ctx_q), quant_scale, batch_size, beam_size, head_num, batch_seq_len,
         hidden, alpha, dequant_scale, current_stream())


def gemm_i8_decode_kernel_16x16(on):
    """Route decode-step products (at most 64 rows) to the 16 x 16 x 64 kernel (default) or to
    the 32 x 32 x 32 one; returns the previous setting."""
    return bool(lib.load().lsh_gemm_i8_decode_kernel_16x16(int(bool(on))))


def dec_emb_norm_layer_i8O(token_emb, pos_emb, tokens, residual, out_q, scale, bias, residual_bias,
                           rows, hidden, vocab_size, step, max_step, dequant_scale, scaled,
                           quant_scale, is_post_ln):
    """Decode step, first layer: target embedding (vocabulary-major int8 table) and the first layer
    norm of the stack in one launch (fp16)."""
    _dev(token_emb, pos_emb, tokens, residual, out_q, scale, bias, residual_bias)
    call("lsh_dec_emb_norm_layer_i8O_f16", ptr(token_emb), ptr(pos_emb), ptr(tokens), ptr(residual),
         ptr(out_q), ptr(scale), ptr(bias), ptr(residual_bias), rows, hidden, vocab_size, step,
         max_step, dequant_scale, int(bool(scaled)), quant_scale, int(bool(is_post_ln)),
         current_stream())


def gpt_emb_step_norm_layer_i8O(token_emb, pos_emb, token_id, residual, out_q, scale, bias,
                                residual_bias, real_seq_len, zero_flag, batch_size, hidden,
                                vocab_size, padding_id, pos, max_step, dequant_scale, quant_scale,
                                is_post_ln):
    """Cached GPT generation step, first layer: the step's token embedding (with the token count
    and the flag clear of the embedding launch) and the first layer norm in one launch (fp16)."""
    _dev(token_emb, pos_emb, token_id, residual, out_q, scale, bias, residual_bias, real_seq_len,
         zero_flag)
    call("lsh_gpt_emb_step_norm_layer_i8O_f16", ptr(token_emb), ptr(pos_emb), ptr(token_id),
         ptr(residual), ptr(out_q), ptr(scale), ptr(bias), ptr(residual_bias), ptr(real_seq_len),
         ptr(zero_flag), batch_size, hidden, vocab_size, padding_id, pos, max_step, dequant_scale,
         quant_scale, int(bool(is_post_ln)), current_stream())


def gemm_i8_tile_kernel(on):
    """Route large products to the one-tile-per-workgroup kernel (default) or to the persistent
    kernels; returns the previous setting."""
    return bool(lib.load().lsh_gemm_i8_tile_kernel(int(bool(on))))


def decself_qkv_attention_in_models(on):
    """Let the generation models fuse the decode-step QKV product with the self attention
    (default) or keep the two launches; returns the previous setting."""
    return bool(lib.load().lsh_decself_qkv_attention_in_models(int(bool(on))))


def bias_act_lut_kernel(on):
    """Let ker_bias_gelu_i8I_i8O tabulate each column's 256 codes in LDS for tensors of 1024
    rows and more (default) or always evaluate per element; returns the previous setting."""
    return bool(lib.load().lsh_bias_act_lut_kernel(int(bool(on))))


def tile_weight_16x64(w, tiled, n, k):
    """[n, k] int8 -> the MFMA-ordered tiling :func:`gemm_i8_residual_ln_i8O` streams."""
    _dev(w, tiled)
    call("lsh_tile_weight_16x64", ptr(w), ptr(tiled), n, k, current_stream())


def gemm_i8_residual_ln_i8O(a, w_tiled, alpha, scale, bias, residual_bias, output, residual,
                            batch_tokens, hidden_size, k, dequant_scale, quant_scale, is_post_ln):
    """Out-projection GEMM + ``ker_residual_bias_ln_i8I_i8O`` in one kernel (fp16)."""
    _dev(a, w_tiled, scale, bias, residual_bias, output, residual)
    call("lsh_gemm_i8_residual_ln_i8O_f16", ptr(a), ptr(w_tiled), alpha, ptr(scale), ptr(bias),
         ptr(residual_bias), ptr(output), ptr(residual), batch_tokens, hidden_size, k,
         dequant_scale, quant_scale, current_stream(), int(bool(is_post_ln)))


def mfma_i8_peak_probe(out, workgroups, iters):
    """Launch the register-resident int8 MFMA loop; returns the integer operations of the launch."""
    import ctypes
    _dev(out)
    ops = ctypes.c_double(0.0)
    call("lsh_mfma_i8_peak_probe", ptr(out), workgroups, iters, ctypes.addressof(ops), current_stream())
    return ops.value


def gemm_i8_lut_i8o(a, w, c, lut, m, n, k, alpha):
    """int8-output GEMM whose epilogue is the table built by :func:`build_act_lut`."""
    _dev(a, w, c, lut)
    call("lsh_gemm_i8_lut_i8o", ptr(a), ptr(w), ptr(c), ptr(lut), m, n, k, alpha, current_stream())


class FfnSegmentSync:
    """Barrier counters, error word and launch count of ``ffn_segment_i8`` (one per caller)."""

    def __init__(self, device="cuda"):
        import ctypes as _c
        L = lib.load()
        L.lsh_ffn_segment_sync_words.restype = _c.c_size_t
        L.lsh_ffn_segment_sync_words.argtypes = []
        self.words = int(L.lsh_ffn_segment_sync_words())
        self.sync = torch.zeros(self.words, dtype=torch.int32, device=device)
        self.launches = _c.c_uint32(0)

    def error(self):
        """The error word after the stream has drained (0 = every wait was met)."""
        return int(self.sync[-1].item()) & 0xFFFFFFFF

    def reset(self):
        self.sync.zero_()
        self.launches.value = 0


def ffn_segment_in_models(on):
    """Let the encoder models run the feed-forward half of a layer as one launch, or as three
    (default); returns the previous setting."""
    return bool(lib.load().lsh_ffn_segment_in_models(int(bool(on))))


def ffn_segment_stamps(buf):
    """Measurement aid: an int64 tensor [256, 8] that every following launch of the segment
    kernel fills with per-workgroup clock values (100 MHz) at its phase boundaries; None: off."""
    if buf is not None and (buf.dtype != torch.int64 or buf.numel() < 256 * 8 or not buf.is_cuda):
        raise ValueError("stamps: an int64 GPU tensor of 256 x 8 values")
    call("lsh_ffn_segment_stamps", ptr(buf))


def ffn_segment_supported(m, hidden, inner):
    return bool(lib.load().lsh_ffn_segment_supported(int(m), int(hidden), int(inner)))


def ffn_segment_i8(x, w1, lut1, alpha1, act, w2, acc, residual, out_t, out_q, scale, bias,
                   residual_bias, colsum, m, hidden, inner, dequant_scale, quant_scale, is_post_ln,
                   final_ln, sync, spin_limit=1 << 15):
    """FFN1 (tabulated epilogue) -> FFN2 -> layer norm of an encoder layer in one launch; ``sync``:
    a :class:`FfnSegmentSync`."""
    import ctypes as _c
    _dev(x, w1, lut1, act, w2, acc, residual, out_t, out_q, scale, bias, residual_bias, colsum)
    call("lsh_ffn_segment_i8_f16", ptr(x), ptr(w1), ptr(lut1), alpha1, ptr(act), ptr(w2), ptr(acc),
         ptr(residual), ptr(out_t), ptr(out_q), ptr(scale), ptr(bias), ptr(residual_bias),
         ptr(colsum), m, hidden, inner, dequant_scale, quant_scale, int(bool(is_post_ln)),
         int(bool(final_ln)), ptr(sync.sync), _c.addressof(sync.launches), int(spin_limit),
         current_stream())
