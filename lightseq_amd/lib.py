"""ctypes binding of ``liblightseq_hip.so``.

``import torch`` happens first on purpose: PyTorch-ROCm ships its own HIP runtime
(SONAME ``libamdhip64.so.7``) and the library must resolve its HIP symbols against
that already-loaded copy so that device pointers and streams are shared.
"""
import ctypes
import os

import torch  # noqa: F401  (must be loaded before the library, see module docstring)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "liblightseq_hip.so")

LSH_OK, LSH_ERR_INVALID, LSH_ERR_UNSUPPORTED, LSH_ERR_HIP, LSH_ERR_IO = range(5)


class LSHError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, code, message, func):
        super().__init__("%s failed (status %d): %s" % (func, code, message))
        self.code = code
        self.func = func


_P, _I, _F, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_long
_CODES = {"p": _P, "s": _P, "i": _I, "f": _F, "l": _L, "c": ctypes.c_char_p, "Q": ctypes.c_uint64}

# name -> (has _f16/_f32 variants, argument codes).  p pointer, s stream, i int, f float,
# l int64_t, Q uint64_t, c C string
_SIGNATURES = {
    "lsh_launch_quantize_tensor": (True, "ppiifsi"),
    "lsh_launch_dequantize_tensor": (True, "ppiifsi"),
    "lsh_ker_norm_layer_resual_i8O": (True, "iispppppifii"),
    "lsh_ker_residual_bias_ln_i32I_i8O": (True, "ppppppiiffisiiip"),
    "lsh_ker_residual_bias_ln_i8I_i8O": (True, "ppppppiiffisiiip"),
    "lsh_ker_residual_bias_ln_i32I": (True, "pppppiifisip"),
    "lsh_ker_bias_gelu_i8I_i8O": (True, "isppp" + "iffii"),
    "lsh_ker_bias_relu_i8I_i8O": (True, "isppp" + "ifffiii"),
    "lsh_ker_arrange_encself_qkv_i8I": (True, "iisppp" + "iiiiifi"),
    "lsh_ker_arrange_encself_qkv_i8I_i8O": (True, "iispppppp" + "iiiiffi"),
    "lsh_ker_arrange_atten_output_i8O": (True, "iispp" + "iiiifi"),
    "lsh_ker_correlation_softmax_encself": (True, "iiispp"),
    "lsh_encself_attention_f16": (False, "pppppp" + "fiiiis"),
    "lsh_encself_attention_i8qkv_f16": (False, "ppfppp" + "fiiiis"),
    "lsh_qkv_attention_i8_f16": (False, "ppppp" + "fff" + "iiiis"),
    "lsh_qkv_attention_plan": (False, "pp" + "iii" + "s"),
    "lsh_qkv_attention_plan_in_models": (False, "i"),
    "lsh_qkv_attention_planned_i8_f16": (False, "pppppp" + "fff" + "iiiis"),
    "lsh_launch_enc_emb_i8I": (True, "ppppp" + "iiiispp" + "ifi"),
    "lsh_launch_scaled_colsum": (True, "ppiifs"),
    "lsh_gemm_i8_i32o": (False, "pppiiis"),
    "lsh_gemm_i8_i8o": (False, "pppiiifs"),
    "lsh_build_act_lut": (False, "pp" + "ifffi" + "s"),
    "lsh_gemm_i8_lut_i8o": (False, "pppp" + "iiif" + "s"),
    "lsh_gemm_i8_decself_qkv_i8o_f16": (False, "pppppp" + "iiiiii" + "fff" + "s"),
    "lsh_decself_qkv_attention_i8_f16": (False, "ppppppp" + "iiiii" + "ffffff" + "s"),
    "lsh_encdec_q_attention_f16": (False, "ppppppp" + "f" + "iiiii" + "ff" + "s"),
    "lsh_gemm_i8_encdec_q_f16": (False, "pppp" + "iiiii" + "ff" + "s"),
    "lsh_gpt_emb_step_norm_layer_i8O_f16": (False, "pppppppppp" + "iiiiii" + "ffi" + "s"),
    "lsh_dec_emb_norm_layer_i8O_f16": (False, "pppppppp" + "iiiii" + "fifi" + "s"),
    "lsh_gemm_i8_i32o_splitk": (False, "ppp" + "iiii" + "p" + "s"),
    "lsh_gemm_i8_preferred_ksplit": (False, "iii"),
    "lsh_layer_norm_row_kernel": (False, "i"),
    "lsh_gemm_i8_tile_kernel": (False, "i"),
    "lsh_gemm_i8_decode_kernel_16x16": (False, "i"),
    "lsh_bias_act_lut_kernel": (False, "i"),
    "lsh_decself_qkv_attention_in_models": (False, "i"),
    "lsh_mfma_i8_peak_probe": (False, "piips"),
    "lsh_ffn_segment_supported": (False, "iii"),
    "lsh_ffn_segment_in_models": (False, "i"),
    "lsh_ffn_segment_stamps": (False, "p"),
    "lsh_ffn_segment_i8_f16": (False, "ppp" + "f" + "ppp" + "ppp" + "pppp" + "iii" + "ff" + "ii" + "pp" +
                               "i" + "s"),
    "lsh_tile_weight_16x64": (False, "ppiis"),
    "lsh_gemm_i8_residual_ln_i8O_f16": (False, "pp" + "f" + "ppppp" + "iii" + "ff" + "s" + "i"),
    "lsh_ker_residual_bias_ln_planes_i32I_i8O_f16": (False, "p" + "il" + "ppppp" + "iiff" + "s" +
                                                     "ip"),
    "lsh_gemm_i8_bias_gelu_i8o_f16": (False, "pppp" + "iiifffs"),
    "lsh_gemm_i8_bias_relu_i8o_f16": (False, "pppp" + "iiiffffis"),
    "lsh_gemm_i8_qkv_arrange_f16": (False, "pppp" + "iiiiiiffs"),
    "lsh_quantize_weight": (True, "ppiifsi"),
    # decoder step
    "lsh_launch_dec_emb_i8I": (True, "pppppp" + "iiiiiii" + "sfi"),
    "lsh_launch_dec_emb_i8I_vocab_major": (True, "pppppp" + "iiiiiii" + "sfi"),
    "lsh_ker_arrange_decself_qkv_i8I_i8O": (True, "iisppppp" + "iiiii" + "ffi"),
    "lsh_decself_scores_i8_i32o": (False, "ppp" + "iiii" + "s"),
    "lsh_ker_fuse_softmax_new_value_i32I_i8O": (False, "ppp" + "iiiii" + "fff" + "is"),
    "lsh_decself_attention_i8": (False, "pppp" + "iiiii" + "fff" + "s"),
    "lsh_ker_arrange_encdec_q_i8I": (True, "iisppp" + "iiii" + "fi"),
    "lsh_ker_arrange_encdec_kv": (True, "iiispppp" + "l" + "iiii"),
    "lsh_ker_correlation_softmax_encdec": (True, "iiispp"),
    "lsh_encdec_attention_f16": (False, "pppppp" + "f" + "iiiii" + "s"),
    "lsh_gemm_f16_nt": (False, "ppp" + "iii" + "s"),
    # beam search
    "lsh_select_beam_rough_topk_i8I": (True, "ppppp" + "f" + "ppp" + "ii" + "f" + "iii" + "s" +
                                       "i" + "f" + "ii"),
    "lsh_ker_refresh_result": (False, "pppppppp" + "ii" + "ff" + "iiii" + "s"),
    "lsh_ker_refresh_cache_i8": (False, "iiis" + "pppppp" + "l" + "iiiiiiii"),
    "lsh_ker_write_trg_tokenid_pos_penalty": (False, "ppp" + "iiii" + "s"),
    "lsh_ker_write_trg_tokenid_neg_penalty": (False, "ppp" + "iiiiii" + "s"),
    "lsh_ker_write_topk_result": (False, "ppp" + "iiiiii" + "s"),
    "lsh_beam_search_step_i8I": (True, "pppppppppp" + "f" + "ii" + "f" + "iiii" + "s"),
    "lsh_beam_search_step_ws_i8I": (True, "pppppppppp" + "f" + "ii" + "f" + "iiii" + "pl" + "s"),
    "lsh_beam_search_step_noalloc_i8I_f16": (False, "pppppppp" + "f" + "ii" + "f" + "iiii" + "s"),
    "lsh_refresh_cache_by_parent_i8": (False, "iis" + "ppppp" + "l" + "iiiii"),
    # GPT path
    "lsh_ker_gpt_embedding_i8I": (True, "iiis" + "ppppp" + "iif"),
    "lsh_gpt_scores_i8_i32o": (False, "ppp" + "iii" + "s"),
    "lsh_ker_correlation_softmax_gpt_i32I": (True, "iiis" + "ppp" + "ff"),
    "lsh_ker_arrange_qkv_with_cache_i8I_i8O": (True, "iis" + "ppppppp" + "iii" + "ffi"),
    "lsh_ker_topk_sample_i8I": (False, "iiiis" + "pppp" + "ii" + "pp" + "ifi"),
    "lsh_ker_ppl_i8I": (False, "iiis" + "pppp" + "ifi"),
    "lsh_ker_ppl_i8I_workspace": (False, "iis" + "pppp" + "if" + "p"),
    "lsh_gpt_arrange_qkv_prefill_f16": (False, "iis" + "ppppppp" + "iiii" + "ff"),
    "lsh_gpt_prefill_attention_f16": (False, "pppppp" + "ff" + "iiii" + "s"),
    "lsh_gpt_prefill_i8_supported": (False, "iii"),
    "lsh_gpt_prefill_on_codes_in_models": (False, "i"),
    "lsh_gpt_arrange_qkv_prefill_i8": (False, "iis" + "ppppp" + "iiii" + "ff"),
    "lsh_gpt_prefill_attention_i8": (False, "ppppp" + "fff" + "iiiii" + "s"),
    "lsh_gpt_greedy_step": (False, "ppp" + "iiii" + "p" + "i" + "s"),
    "lsh_gpt_sample_step": (False, "ppp" + "iiii" + "p" + "i" + "iff" + "p" + "s"),
    "lsh_ker_topp_sample_i8I": (False, "iiiis" + "pppp" + "if" + "pp" + "ifi"),
    "lsh_rng_setup": (False, "piQs"),
    "lsh_ker_topk_sample_i8I_dec": (True, "iiiiis" + "pppp" + "ii" + "pp" + "ifi"),
    "lsh_ker_topp_sample_i8I_dec": (True, "iiiiis" + "pppp" + "if" + "pp" + "ifi"),
    "lsh_ker_attention_mask_weights_i32I": (True, "iiiis" + "ppp" + "ff"),
    # operator launchers of the csrc layer path (include/lightseq_ops.h)
    "lsh_launch_quantize": (True, "ppppp" + "ii" + "s"),
    "lsh_launch_quantize_2d": (True, "ppppp" + "iii" + "s" + "i"),
    "lsh_launch_fake_quantize": (True, "ppppp" + "ii" + "s" + "i"),
    "lsh_launch_dequantize": (True, "ppp" + "ii" + "s"),
    "lsh_launch_layer_norm": (True, "pppppp" + "ii" + "s"),
    "lsh_launch_layer_norm_i8": (True, "pppppppp" + "ii" + "s"),
    "lsh_launch_attn_softmax": (True, "pp" + "iiiii" + "s"),
    "lsh_launch_quant_bias_add_transform_20314": (True, "ppppp" + "iiiii" + "s" + "p" + "i"),
    "lsh_launch_bias_add_transform_20314": (True, "ppp" + "iiiii" + "s"),
    "lsh_launch_concat3_dim1": (True, "ppp" + "iiii" + "s"),
    "lsh_launch_transform4d_0213": (True, "pp" + "iiiii" + "s"),
    "lsh_launch_quant_transform4d_0213": (True, "pppp" + "iiiii" + "s"),
    "lsh_launch_ls_dropout": (True, "ppp" + "if" + "s" + "i"),
    "lsh_launch_ls_dropout_res_bias": (True, "ppppp" + "iif" + "s"),
    "lsh_launch_ls_dropout_act_bias_gelu": (True, "pppp" + "iif" + "s"),
    "lsh_launch_ls_dropout_act_bias_relu": (True, "pppp" + "iif" + "s"),
    "lsh_launch_ls_quant_dropout_act_bias_gelu": (True, "pppppppp" + "iif" + "s"),
    "lsh_launch_ls_quant_dropout_act_bias_relu": (True, "pppppppp" + "iif" + "s"),
    "lsh_launch_ls_fakequant_dropout_act_bias_gelu": (True, "pppppppp" + "iif" + "s" + "ii"),
    "lsh_launch_ls_fakequant_dropout_act_bias_relu": (True, "pppppppp" + "iif" + "s" + "ii"),
    "lsh_launch_ls_quant_dropout_res_bias": (True, "pppppp" + "iif" + "s" + "i"),
    "lsh_feed_forward_i8": (False, "iii" + "ppppp" + "s"),
    "lsh_strided_batch_gemm": (True, "iiii" + "ff" + "ii" + "ppp" + "s"),
    "lsh_layer_attention_f16": (False, "ppppp" + "iiiii" + "s"),
    "lsh_layer_cross_attention_f16": (False, "ppppp" + "iiiiii" + "s"),
    # layer interface
    "ls_layer_set_stream": (False, "s"),
    "ls_create_transformer_encoder_layer_fp16": (False, "iiiiii" + "fff" + "i" + "c" + "i"),
    "ls_transformer_encoder_layer_fw_fp16": (False, "i" + "ppp" + "iiiii"),
    "ls_create_transformer_decoder_layer_fp16": (False, "iiiiii" + "fff" + "i" + "c"),
    "ls_transformer_decoder_layer_fw_fp16": (False, "i" + "pppp" + "iiii" + "p" + "iii"),
    "ls_layer_param_count": (False, "c" + "i" + "p"),
    "ls_assign_layer_weight_grad_fp16": (False, "pp" + "c" + "i"),
    "ls_create_quant_linear_layer_fp16": (False, "iiii"),
    "ls_quant_linear_layer_fw_fp16": (False, "i" + "pppp" + "iii"),
    "ls_destroy_layer": (False, "c" + "i"),
}

_lib = None


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing: build it with `python -m lightseq_amd.build` "
            "(there is no CPU fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    lib.lsh_last_error.restype = ctypes.c_char_p
    lib.lsh_last_error.argtypes = []
    lib.lsh_version.restype = ctypes.c_char_p
    lib.lsh_version.argtypes = []
    lib.lsh_length_norm.restype = ctypes.c_float
    lib.lsh_length_norm.argtypes = [_I, _F]
    for name, (typed, codes) in _SIGNATURES.items():
        for suffix in (("_f16", "_f32") if typed else ("",)):
            fn = getattr(lib, name + suffix)
            fn.restype = ctypes.c_int
            fn.argtypes = [_CODES[c] for c in codes]
    _lib = lib
    return lib


def bind(name, codes, restype=ctypes.c_int):
    """Declare one more entry point (used by modules that add their own)."""
    fn = getattr(load(), name)
    fn.restype = restype
    fn.argtypes = [_CODES[c] for c in codes]
    return fn


def last_error():
    return load().lsh_last_error().decode()


def version():
    return load().lsh_version().decode()


def ptr(x):
    """Device pointer of a torch tensor (None -> NULL); ints pass through."""
    if x is None:
        return None
    if isinstance(x, torch.Tensor):
        if not x.is_contiguous():
            raise ValueError("tensor must be contiguous")
        return x.data_ptr()
    return int(x)


def current_stream():
    return torch.cuda.current_stream().cuda_stream


def call(name, *args):
    """Call ``name`` and raise :class:`LSHError` on a non-zero status."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise LSHError(rc, lib.lsh_last_error().decode(), name)
