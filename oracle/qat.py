"""CPU restatement (numpy) of the reference's pure-PyTorch quantisation-aware encoder layer:
``TransformerEncoderLayer`` (training/ops/pytorch/torch_transformer_layers.py:537-679) with
``MultiheadAttention`` (:36-396), ``QuantLinear`` (training/ops/pytorch/quantization.py:33-62)
and ``_tensor_quant`` (training/pytorch_quantization/tensor_quant.py:349-409).

TEST INFRASTRUCTURE ONLY: imported by ``tests/`` -- never by the shipped package.

This is the fake-quantised ("QAT form") layer the int8 kernels are trained against: every
``QuantLinear`` is  fq(input) -> fq(weight) -> linear without bias -> fq(output) -> + bias,
attention and layer norm are float.  Everything here is float32 numpy; the reference module
was read, not imported.
"""
import numpy as np
from scipy.special import erf

F32 = np.float32


def tensor_quant(x, amax, num_bits=8, unsigned=False, narrow_range=True):
    """tensor_quant.py:349-409 ``_tensor_quant``: returns (integer-valued float32, scale)."""
    x = np.asarray(x, F32)
    amax = F32(amax)
    max_bound = F32(2.0 ** (num_bits - 1) - 1.0)
    min_bound = -max_bound if narrow_range else -max_bound - 1
    scale = amax / (max_bound * 2) if unsigned else amax / max_bound
    if amax <= 1.0 / (1 << 24):
        return np.zeros_like(x), F32(1.0)
    out = x / scale
    if unsigned:
        out = out - max_bound
    out = np.floor(out + F32(0.5))
    return np.clip(out, min_bound, max_bound).astype(F32), scale


def fake_tensor_quant(x, amax, unsigned=False):
    """tensor_quant.py:328-346 ``FakeTensorQuantFunction.forward``."""
    q, scale = tensor_quant(x, amax, 8, unsigned, True)
    if unsigned:
        q = q + F32(127.0)
    return (q * scale).astype(F32)


def tensor_quantizer(x, amax, learn_amax, unsigned=False, enabled=True):
    """nn/modules/tensor_quantizer.py:340-398: an optional clip to [-amax, amax]
    (``learn_amax``; nn/modules/clip.py:75-78) followed by the fake quantisation."""
    if not enabled:
        return np.asarray(x, F32)
    x = np.asarray(x, F32)
    if unsigned and x.min() < 0:
        raise TypeError("Negative values encountered in unsigned quantization.")
    if learn_amax:
        x = np.clip(x, -F32(amax), F32(amax))
    return fake_tensor_quant(x, amax, unsigned)


def quant_linear(x, weight, bias, in_amax, w_amax, out_amax, pre_activation=None, quant=True,
                 output_quant=True):
    """quantization.py:33-62 ``QuantLinear.forward``.  ``pre_activation="relu"`` selects the
    unsigned input quantiser (:22-24,36-39)."""
    qx = tensor_quantizer(x, in_amax, True, pre_activation == "relu", quant)
    qw = tensor_quantizer(weight, w_amax, False, False, quant)
    out = qx @ qw.T
    out = tensor_quantizer(out, out_amax, False, False, quant and output_quant)
    if bias is not None:
        out = out + np.asarray(bias, F32)
    return out.astype(F32)


def layer_norm(x, w, b, eps=1e-5):
    x = np.asarray(x, np.float64)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return ((x - mu) / np.sqrt(var + eps) * np.asarray(w, np.float64)
            + np.asarray(b, np.float64)).astype(F32)


def activation(x, name):
    """util.py:14-30: relu, or the erf GELU of torch.nn.functional.gelu."""
    if name == "relu":
        return np.maximum(x, F32(0))
    if name == "gelu":
        x64 = np.asarray(x, np.float64)
        return (0.5 * x64 * (1.0 + erf(x64 / np.sqrt(2.0)))).astype(F32)
    raise RuntimeError("--activation-fn {} not supported".format(name))


def self_attention(x, p, amax, nhead, key_padding_mask, quant=True):
    """torch_transformer_layers.py:151-376 for self attention without incremental state.
    x: [T, B, C] (time first, as the module receives it)."""
    tgt, bsz, c = x.shape
    hd = c // nhead
    qkv = quant_linear(x, p["qkv_w"], p["qkv_b"], amax["qkv_in"], amax["qkv_w"], amax["qkv_out"],
                       quant=quant)
    q, k, v = np.split(qkv, 3, axis=-1)
    q = q * F32(hd ** -0.5)
    q = q.reshape(tgt, bsz * nhead, hd).transpose(1, 0, 2)
    k = k.reshape(tgt, bsz * nhead, hd).transpose(1, 0, 2)
    v = v.reshape(tgt, bsz * nhead, hd).transpose(1, 0, 2)
    w = (q @ k.transpose(0, 2, 1)).astype(F32)
    if key_padding_mask is not None:
        w = w.reshape(bsz, nhead, tgt, tgt)
        w = np.where(np.asarray(key_padding_mask, bool)[:, None, None, :], -np.inf, w)
        w = w.reshape(bsz * nhead, tgt, tgt)
    w = w - w.max(-1, keepdims=True)
    e = np.exp(w.astype(np.float64))
    probs = (e / e.sum(-1, keepdims=True)).astype(F32)
    attn = (probs @ v).transpose(1, 0, 2).reshape(tgt, bsz, c)
    return quant_linear(attn, p["out_w"], p["out_b"], amax["out_in"], amax["out_w"],
                        amax["out_out"], quant=quant)


def encoder_layer(x, p, amax, nhead, pre_ln, act, key_padding_mask=None, quant=True,
                  fc2_output_quant=True):
    """torch_transformer_layers.py:630-679 ``TransformerEncoderLayer.forward`` in eval mode.

    x: [B, S, H]; p: dict of qkv_w [3H,H], qkv_b, out_w, out_b, ln1_w, ln1_b, fc1_w [I,H],
    fc1_b, fc2_w [H,I], fc2_b, ln2_w, ln2_b; amax: dict of the twelve clip values
    (qkv_in, qkv_w, qkv_out, out_in, out_w, out_out, fc1_in, fc1_w, fc1_out, fc2_in, fc2_w,
    fc2_out).  ``fc2_output_quant=False`` switches the output quantiser of fc2 off (the
    module's own ``disable_quant``): the int8 kernels do not quantise that output."""
    x = np.asarray(x, F32).transpose(1, 0, 2)
    residual = x
    if pre_ln:
        x = layer_norm(x, p["ln1_w"], p["ln1_b"])
    x = self_attention(x, p, amax, nhead, key_padding_mask, quant)
    x = residual + x
    if not pre_ln:
        x = layer_norm(x, p["ln1_w"], p["ln1_b"])
    residual = x
    if pre_ln:
        x = layer_norm(x, p["ln2_w"], p["ln2_b"])
    x = activation(quant_linear(x, p["fc1_w"], p["fc1_b"], amax["fc1_in"], amax["fc1_w"],
                                amax["fc1_out"], quant=quant), act)
    x = quant_linear(x, p["fc2_w"], p["fc2_b"], amax["fc2_in"], amax["fc2_w"], amax["fc2_out"],
                     pre_activation=act, quant=quant, output_quant=fc2_output_quant)
    x = residual + x
    if not pre_ln:
        x = layer_norm(x, p["ln2_w"], p["ln2_b"])
    return x.transpose(1, 0, 2).astype(F32)
