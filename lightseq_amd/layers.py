"""Layer classes over the layer C ABI (``include/lightseq_ops.h``), mirroring the reference's
``LSTransformerEncoderLayer`` (lightseq/training/ops/pytorch/transformer_encoder_layer.py:82-352),
``LSTransformerDecoderLayer`` (training/ops/pytorch/transformer_decoder_layer.py:112-537) and
``LSQuantLinearLayer``: one flat parameter tensor per layer holding the weights, biases,
layer-norm parameters and the clip values; ``forward(hidden_states, padding_mask)``.

Forward only, fp16, quantised mode (call :meth:`enable_quant`, as with the reference, and put
the module in ``eval()`` mode).  torch owns the parameter and activation memory; the layer
computes with the library's HIP kernels on torch's current stream.
"""
import copy
import ctypes
import itertools
import math
from dataclasses import dataclass

import torch
from torch import nn

from .lib import call, current_stream, ptr

# default clip values of the reference (training/ops/pytorch/quantization.py:14-25)
ACT_CLIP_MAX = 16.0
WEIGHT_CLIP_MAX = 1.0

_layer_ids = itertools.count()


def calc_offset(sizes):
    """training/ops/pytorch/util.py:65-71."""
    offsets = [0]
    for x in sizes:
        offsets.append(offsets[-1] + x)
    return offsets


class LSTransformerEncoderLayer(nn.Module):
    @staticmethod
    def get_config(**kwargs):
        """training/ops/pytorch/layer_base.py:9-34."""

        @dataclass
        class Config:
            max_batch_tokens: int
            max_seq_len: int
            hidden_size: int
            intermediate_size: int
            nhead: int
            attn_prob_dropout_ratio: float
            activation_dropout_ratio: float
            hidden_dropout_ratio: float
            pre_layer_norm: bool
            fp16: bool
            local_rank: int
            activation_fn: str = "relu"

        return Config(**kwargs)

    @staticmethod
    def gen_offset(hidden_size, intermediate_size):
        """transformer_encoder_layer.py:153-172."""
        hs, ims = hidden_size, intermediate_size
        return calc_offset([hs * hs * 3, hs * 3, hs * hs, hs, hs, hs, hs * ims, ims, hs * ims, hs,
                            hs, hs, 12])

    def __init__(self, config, initial_weights=None, initial_biases=None):
        super().__init__()
        if not config.fp16:
            raise ValueError("only the fp16 layer is provided")
        self.config = config
        self.layer_id = next(_layer_ids)
        self.quant_mode = False
        self.hs, self.ims = config.hidden_size, config.intermediate_size
        call("ls_create_transformer_encoder_layer_fp16", self.layer_id, config.max_batch_tokens,
             config.max_seq_len, config.hidden_size, config.nhead, config.intermediate_size,
             config.attn_prob_dropout_ratio, config.activation_dropout_ratio,
             config.hidden_dropout_ratio, int(config.pre_layer_norm),
             config.activation_fn.encode(), 0)
        self.para_offset = self.gen_offset(self.hs, self.ims)
        self.para = nn.Parameter(torch.zeros(self.para_offset[-1]))
        if initial_weights is None or initial_biases is None:
            self.init_transformer_weights()
        else:
            # the reference's test hook: lists [q, k, v, out, ln1, fc1, fc2, ln2]
            ws = [torch.cat([w.detach() for w in initial_weights[:3]], 0)] + list(initial_weights[3:])
            bs = [torch.cat([b.detach() for b in initial_biases[:3]], 0)] + list(initial_biases[3:])
            for i, (w, b) in enumerate(zip(ws, bs)):
                self._get_weights(2 * i).copy_(w.detach().reshape(-1))
                self._get_weights(2 * i + 1).copy_(b.detach().reshape(-1))
            self._init_clip_max()

    def _get_weights(self, i):
        return self.para.data.narrow(0, self.para_offset[i],
                                     self.para_offset[i + 1] - self.para_offset[i])

    def _init_clip_max(self):
        self._get_weights(12).copy_(
            torch.tensor([ACT_CLIP_MAX, WEIGHT_CLIP_MAX, ACT_CLIP_MAX] * 4))

    def init_transformer_weights(self):
        """transformer_encoder_layer.py:212-242."""
        hs, ims = self.hs, self.ims

        def bound(w):
            return 1.0 / math.sqrt(w.shape[1])

        qkvw = self._get_weights(0).view(-1, hs)
        nn.init.xavier_uniform_(qkvw, 1.0 / math.sqrt(2.0))
        nn.init.uniform_(self._get_weights(1), -bound(qkvw), bound(qkvw))
        nn.init.xavier_uniform_(self._get_weights(2).view(-1, hs), 1.0)
        nn.init.zeros_(self._get_weights(3))
        nn.init.ones_(self._get_weights(4))
        nn.init.zeros_(self._get_weights(5))
        inter_w = self._get_weights(6).view(ims, hs)
        nn.init.kaiming_uniform_(inter_w, math.sqrt(5.0))
        nn.init.uniform_(self._get_weights(7), -bound(inter_w), bound(inter_w))
        output_w = self._get_weights(8).view(hs, ims)
        nn.init.kaiming_uniform_(output_w, math.sqrt(5.0))
        nn.init.uniform_(self._get_weights(9), -bound(output_w), bound(output_w))
        nn.init.ones_(self._get_weights(10))
        nn.init.zeros_(self._get_weights(11))
        self._init_clip_max()

    def enable_quant(self):
        self.quant_mode = True

    def disable_quant(self):
        self.quant_mode = False

    def forward(self, hidden_states, encoder_padding_mask, **kwargs):
        """hidden_states [batch, seq_len, hidden]; encoder_padding_mask [batch, seq_len] with
        1 for padding and 0 for tokens (transformer_encoder_layer.py:309-352)."""
        if not hidden_states.is_cuda:
            raise ValueError("the layer runs on the GPU only (no CPU fallback exists)")
        hidden_states = hidden_states.contiguous().to(torch.half)
        mask = (encoder_padding_mask * -1e8).to(torch.half).contiguous()
        para = self.para if self.para.dtype == torch.half else self._half_para()
        bs, sl, dim = hidden_states.size()
        if bs * sl > self.config.max_batch_tokens:
            raise ValueError(f"Batch token numbers {bs * sl} exceeds the limit"
                             f" {self.config.max_batch_tokens}.")
        if sl > self.config.max_seq_len:
            raise ValueError(f"Sequence length {sl} exceeds the limit {self.config.max_seq_len}.")
        if mask.dim() == 1:
            assert bs == 1 and sl == mask.size(0)
        else:
            assert bs == mask.size(0) and sl == mask.size(1)
        call("ls_layer_set_stream", current_stream())
        call("ls_assign_layer_weight_grad_fp16", ptr(para), None, b"TransformerEncoderLayer",
             self.layer_id)
        output = torch.empty_like(hidden_states)
        call("ls_transformer_encoder_layer_fw_fp16", self.layer_id, ptr(hidden_states), ptr(mask),
             ptr(output), bs, sl, int(self.training), int(self.config.pre_layer_norm),
             int(self.quant_mode))
        return output.to(self.para.dtype)

    def _half_para(self):
        if not hasattr(self, "para_16"):
            self.register_buffer("para_16", self.para.detach().clone().half(), persistent=False)
        else:
            self.para_16.copy_(self.para.detach().to(torch.half))
        return self.para_16

    def __del__(self):
        try:
            call("ls_destroy_layer", b"TransformerEncoderLayer", self.layer_id)
        except Exception:
            pass


class LSTransformerDecoderLayer(nn.Module):
    """Decoder layer: self attention (cached in a decoding step), cross attention over the
    encoder output, feed-forward.  Layer 0 of a stack also owns the cross-attention k/v
    projection of every layer, so ``config.nlayer`` layers must be created, in order, before
    the first forward call."""

    layer_id = 0  # class counter, as in the reference (transformer_decoder_layer.py:126-133)

    @staticmethod
    def get_config(**kwargs):
        """training/ops/pytorch/layer_base.py:49-76."""

        @dataclass
        class Config:
            max_batch_tokens: int
            max_seq_len: int
            hidden_size: int
            intermediate_size: int
            nhead: int
            attn_prob_dropout_ratio: float
            activation_dropout_ratio: float
            hidden_dropout_ratio: float
            pre_layer_norm: bool
            fp16: bool
            local_rank: int
            nlayer: int
            activation_fn: str = "relu"

        return Config(**kwargs)

    @classmethod
    def new_stack(cls):
        """Starts counting layers at 0 again, for a second decoder in one process (the
        reference builds one per process).  A layer created under an id that is in use
        replaces the old one."""
        cls.layer_id = 0

    @staticmethod
    def gen_offset(hidden_size, intermediate_size, nlayer):
        """transformer_decoder_layer.py:208-238."""
        hs, ims = hidden_size, intermediate_size
        return calc_offset([hs * hs * 3, hs * 3, hs * hs, hs, hs, hs,
                            hs * hs, hs, hs * hs, hs, hs, hs,
                            hs * ims, ims, hs * ims, hs, hs, hs,
                            24, hs * hs * 2 * nlayer, hs * 2 * nlayer])

    def __init__(self, config, initial_weights=None, initial_biases=None):
        super().__init__()
        if not config.fp16:
            raise ValueError("only the fp16 layer is provided")
        self.config = copy.deepcopy(config)
        self.config.layer_id = LSTransformerDecoderLayer.layer_id
        LSTransformerDecoderLayer.layer_id += 1
        self.quant_mode = False
        self.hs, self.ims = config.hidden_size, config.intermediate_size
        call("ls_create_transformer_decoder_layer_fp16", self.config.layer_id,
             config.max_batch_tokens, config.max_seq_len, config.hidden_size, config.nhead,
             config.intermediate_size, config.attn_prob_dropout_ratio,
             config.activation_dropout_ratio, config.hidden_dropout_ratio,
             int(config.pre_layer_norm), config.activation_fn.encode())
        self.para_offset = self.gen_offset(self.hs, self.ims, config.nlayer)
        if self.config.layer_id != 0:
            self.para_offset = self.para_offset[:-2]
        self.para = nn.Parameter(torch.zeros(self.para_offset[-1]))
        if initial_weights is None or initial_biases is None:
            self.init_transformer_weights()
            return
        # the reference's test hook (transformer_decoder_layer.py:181-205): q, k, v first, then
        # weights and biases alternate, None entries skipped
        ws = [torch.cat([w.detach() for w in initial_weights[:3]], 0)] + list(initial_weights[3:])
        bs = [torch.cat([b.detach() for b in initial_biases[:3]], 0)] + list(initial_biases[3:])
        idx = 0
        for w, b in itertools.zip_longest(ws, bs):
            for t in (w, b):
                if t is not None:
                    cur = self._get_weights(idx)
                    assert cur.numel() == t.numel()
                    cur.copy_(t.detach().reshape(-1))
                    idx += 1

    def _get_weights(self, i):
        return self.para.data.narrow(0, self.para_offset[i],
                                     self.para_offset[i + 1] - self.para_offset[i])

    def init_transformer_weights(self):
        """transformer_decoder_layer.py:325-375."""
        hs, ims = self.hs, self.ims

        def bound(w):
            return 1.0 / math.sqrt(w.shape[1])

        qkvw = self._get_weights(0).view(-1, hs)
        nn.init.xavier_uniform_(qkvw, 1.0 / math.sqrt(2.0))
        nn.init.uniform_(self._get_weights(1), -bound(qkvw), bound(qkvw))
        qw = self._get_weights(6).view(hs, hs)
        nn.init.xavier_uniform_(qw, 1.0 / math.sqrt(2.0))
        nn.init.uniform_(self._get_weights(7), -bound(qw), bound(qw))
        for i in (2, 8):
            nn.init.xavier_uniform_(self._get_weights(i).view(hs, hs), 1.0)
            nn.init.zeros_(self._get_weights(i + 1))
        inter_w = self._get_weights(12).view(ims, hs)
        nn.init.kaiming_uniform_(inter_w, math.sqrt(5.0))
        nn.init.uniform_(self._get_weights(13), -bound(inter_w), bound(inter_w))
        output_w = self._get_weights(14).view(hs, ims)
        nn.init.kaiming_uniform_(output_w, math.sqrt(5.0))
        nn.init.uniform_(self._get_weights(15), -bound(output_w), bound(output_w))
        for i in (4, 10, 16):
            nn.init.ones_(self._get_weights(i))
            nn.init.zeros_(self._get_weights(i + 1))
        self._get_weights(18).copy_(
            torch.tensor([ACT_CLIP_MAX, WEIGHT_CLIP_MAX, ACT_CLIP_MAX] * 8))
        if self.config.layer_id == 0:
            kvw = self._get_weights(19).view(-1, hs)
            nn.init.xavier_uniform_(kvw, 1.0 / math.sqrt(2.0))
            nn.init.uniform_(self._get_weights(20), -bound(kvw), bound(kvw))

    def enable_quant(self):
        self.quant_mode = True

    def disable_quant(self):
        self.quant_mode = False

    def forward(self, decoder_states, encoder_out, encoder_padding_mask, cache=None, **kwargs):
        """decoder_states [batch, trg_len, hidden], or [batch * beam, 1, hidden] in a decoding
        step; encoder_out [src_len, batch, hidden]; encoder_padding_mask [batch, src_len], 1 for
        padding; cache: None, or a dict that the layer fills and updates: ``dec_self_k`` /
        ``dec_self_v`` [batch * beam, heads, step, head_dim] and, on layer 0, ``encdec_kv``
        [layers * 2, batch, src_len * hidden] (transformer_decoder_layer.py:426-531)."""
        if not decoder_states.is_cuda:
            raise ValueError("the layer runs on the GPU only (no CPU fallback exists)")
        decoder_states = decoder_states.contiguous().to(torch.half)
        encoder_out = encoder_out.transpose(0, 1).contiguous().to(torch.half)
        mask = (encoder_padding_mask * -1e8).to(torch.half).contiguous()
        para = self.para if self.para.dtype == torch.half else self._half_para()
        cfg = self.config
        step, cache_list = -1, None
        if cache is not None:
            batch_beams = decoder_states.shape[0]
            old = [None, None]
            if cache:
                step = cache["dec_self_k"].shape[2]
                old = [cache["dec_self_k"].contiguous(), cache["dec_self_v"].contiguous()]
            else:
                step = 0
            encdec_kv = None
            if cfg.layer_id == 0:
                if step == 0:
                    cache["encdec_kv"] = torch.zeros(
                        (cfg.nlayer * 2, encoder_out.shape[0], encoder_out.shape[1] * self.hs),
                        dtype=torch.half, device=decoder_states.device)
                encdec_kv = cache["encdec_kv"]
            shape = (batch_beams, cfg.nhead, step + 1, self.hs // cfg.nhead)
            new_k = torch.zeros(shape, dtype=torch.half, device=decoder_states.device)
            new_v = torch.zeros(shape, dtype=torch.half, device=decoder_states.device)
            cache_list = [new_k, new_v] + old + [encdec_kv]
            cache["dec_self_k"], cache["dec_self_v"] = new_k, new_v
        bs, sl, dim = decoder_states.size()
        if bs * sl > cfg.max_batch_tokens:
            raise ValueError(f"Batch token numbers {bs * sl} exceeds the limit"
                             f" {cfg.max_batch_tokens}.")
        if sl > cfg.max_seq_len:
            raise ValueError(f"Sequence length {sl} exceeds the limit {cfg.max_seq_len}.")
        if mask.dim() == 1:
            assert encoder_out.size(0) == 1 and encoder_out.size(1) == mask.size(0)
        else:
            assert encoder_out.size(0) == mask.size(0) and encoder_out.size(1) == mask.size(1)
        batch = encoder_out.size(0)
        if cache is None:
            assert bs == batch
            trg_len = sl
        else:
            assert bs % batch == 0 and sl == 1
            trg_len = bs // batch  # the beam size
        call("ls_layer_set_stream", current_stream())
        call("ls_assign_layer_weight_grad_fp16", ptr(para), None, b"TransformerDecoderLayer",
             cfg.layer_id)
        output = torch.empty_like(decoder_states)
        cache_ptrs = None
        if cache_list is not None:
            cache_ptrs = (ctypes.c_void_p * 5)(*[ptr(t) for t in cache_list])
        training = self.training and cache is None
        call("ls_transformer_decoder_layer_fw_fp16", cfg.layer_id, ptr(decoder_states),
             ptr(encoder_out), ptr(mask), ptr(output), batch, trg_len, encoder_out.size(1), step,
             cache_ptrs, int(training), int(cfg.pre_layer_norm), int(self.quant_mode))
        return output.to(self.para.dtype)

    def _half_para(self):
        if not hasattr(self, "para_16"):
            self.register_buffer("para_16", self.para.detach().clone().half(), persistent=False)
        else:
            self.para_16.copy_(self.para.detach().to(torch.half))
        return self.para_16

    def release(self):
        """Frees the layer's device buffers (the reference keeps them until the process ends).
        Not done on garbage collection: a later stack may reuse the id."""
        call("ls_destroy_layer", b"TransformerDecoderLayer", self.config.layer_id)


class LSQuantLinearLayer(nn.Module):
    """``outputs = dequantize(int8_gemm(quantize(inputs), quantize(weight)))`` with three
    clip values (input, weight, output), lightseq/csrc/layers/quant_linear_layer.cpp:22-45."""

    def __init__(self, in_features, out_features, max_batch_tokens):
        super().__init__()
        self.layer_id = next(_layer_ids)
        self.in_features, self.out_features = in_features, out_features
        self.max_batch_tokens = max_batch_tokens
        call("ls_create_quant_linear_layer_fp16", self.layer_id, in_features, out_features,
             max_batch_tokens)
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        nn.init.kaiming_uniform_(self.weight, math.sqrt(5.0))
        self.clip_max = nn.Parameter(torch.tensor([ACT_CLIP_MAX, WEIGHT_CLIP_MAX, ACT_CLIP_MAX]))

    def forward(self, inputs):
        if not inputs.is_cuda:
            raise ValueError("the layer runs on the GPU only (no CPU fallback exists)")
        x = inputs.contiguous().to(torch.half)
        tokens = x.numel() // self.in_features
        w = self.weight.detach().to(torch.half).contiguous()
        cm = self.clip_max.detach().to(torch.half).contiguous()
        out = torch.empty(*x.shape[:-1], self.out_features, dtype=torch.half, device=x.device)
        call("ls_layer_set_stream", current_stream())
        call("ls_quant_linear_layer_fw_fp16", self.layer_id, ptr(x), ptr(w), ptr(cm), ptr(out),
             tokens, 1, 1)
        return out

    def __del__(self):
        try:
            call("ls_destroy_layer", b"QuantLinearLayer", self.layer_id)
        except Exception:
            pass
