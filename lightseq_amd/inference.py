"""``lightseq.inference``-style model classes over the model C ABI.

Mirrors the pybind classes of the reference
(lightseq/inference/pywrapper/wrapper.cc:85-156 ``PyQuantTransformer``, :240-320
``PyQuantBert``): the constructor
takes ``(weight_path, max_batch_size)``, ``infer`` takes a C-contiguous int32
``[batch, seq_len]`` numpy array, copies it to the device, runs the model and
returns the output as a float32 numpy array.  Device buffers are allocated once at
the model's maximum shapes, as the reference does; torch is used only to own that
device memory.
"""
import ctypes

import numpy as np
import torch

from . import lib

_P, _I = ctypes.c_void_p, ctypes.c_int
_LS_MAX_DIMS = 8

_NP_OF_DTYPE = {1: np.float32, 2: np.int32, 4: np.float16}
_TORCH_OF_DTYPE = {1: torch.float32, 2: torch.int32, 4: torch.float16}

_bound = False


def _bind():
    global _bound
    if _bound:
        return lib.load()
    L = lib.load()
    pp = ctypes.POINTER(_P)
    ip = ctypes.POINTER(_I)
    sigs = {
        "ls_model_create": [ctypes.c_char_p, ctypes.c_char_p, _I, pp],
        "ls_model_destroy": [_P],
        "ls_model_infer": [_P],
        "ls_model_set_input_ptr": [_P, _I, _P],
        "ls_model_set_input_shape": [_P, _I, ip, _I],
        "ls_model_get_input_max_shape": [_P, _I, ip, ip],
        "ls_model_get_input_size": [_P, ip],
        "ls_model_get_input_name": [_P, _I, ctypes.POINTER(ctypes.c_char_p)],
        "ls_model_get_input_dtype": [_P, _I, ip],
        "ls_model_set_output_ptr": [_P, _I, _P],
        "ls_model_get_output_ptr": [_P, _I, pp],
        "ls_model_get_output_size": [_P, ip],
        "ls_model_get_output_name": [_P, _I, ctypes.POINTER(ctypes.c_char_p)],
        "ls_model_get_output_shape": [_P, _I, ip, ip],
        "ls_model_get_output_max_shape": [_P, _I, ip, ip],
        "ls_model_get_output_dtype": [_P, _I, ip],
        "ls_model_benchmark_mode": [_P, _I],
        "ls_model_get_stream": [_P, pp],
        "ls_model_set_tap": [_P, _I, ctypes.c_char_p, _P],
        "ls_model_set_tap_step": [_P, _I],
        "ls_model_set_profiling": [_P, _I],
        "ls_model_get_profile": [_P, ctypes.c_char_p, _I],
        "ls_model_get_phase_times": [_P, _P, _P, _P],
        "ls_model_set_step_record": [_P, _P, _P, _I],
        "ls_model_get_steps_run": [_P, ip],
        "ls_model_set_graph_mode": [_P, _I],
        "ls_model_set_seed": [_P, ctypes.c_uint64],
        "ls_model_get_graph_stats": [_P, ip, ctypes.POINTER(ctypes.c_longlong)],
        "ls_model_get_graph_nodes": [_P, ip],
    }
    for name, argtypes in sigs.items():
        fn = getattr(L, name)
        fn.restype = _I
        fn.argtypes = argtypes
    _bound = True
    return L


class LSModel:
    """Thin object over an ``ls_model*`` handle (LSModel of the reference)."""

    def __init__(self, class_name, weight_path, max_batch_size):
        self._lib = _bind()
        self._h = _P()
        self._call("ls_model_create", class_name.encode(), str(weight_path).encode(),
                   int(max_batch_size), ctypes.byref(self._h))

    def _call(self, name, *args):
        rc = getattr(self._lib, name)(*args)
        if rc != 0:
            raise lib.LSHError(rc, self._lib.lsh_last_error().decode(), name)

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            self._lib.ls_model_destroy(self._h)
            self._h = _P()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- LSModel methods ------------------------------------------------------
    def infer_device(self):
        self._call("ls_model_infer", self._h)

    def set_input_ptr(self, index, ptr):
        self._call("ls_model_set_input_ptr", self._h, index, _P(ptr))

    def set_input_shape(self, index, shape):
        arr = (_I * len(shape))(*[int(s) for s in shape])
        self._call("ls_model_set_input_shape", self._h, index, arr, len(shape))

    def _shape(self, fn, index):
        arr = (_I * _LS_MAX_DIMS)()
        n = _I()
        self._call(fn, self._h, index, arr, ctypes.byref(n))
        return [arr[i] for i in range(n.value)]

    def get_input_max_shape(self, index):
        return self._shape("ls_model_get_input_max_shape", index)

    def get_output_max_shape(self, index):
        return self._shape("ls_model_get_output_max_shape", index)

    def get_output_shape(self, index):
        return self._shape("ls_model_get_output_shape", index)

    def _int(self, fn, *args):
        v = _I()
        self._call(fn, self._h, *args, ctypes.byref(v))
        return v.value

    def get_input_size(self):
        return self._int("ls_model_get_input_size")

    def get_output_size(self):
        return self._int("ls_model_get_output_size")

    def get_input_dtype(self, index):
        return self._int("ls_model_get_input_dtype", index)

    def get_output_dtype(self, index):
        return self._int("ls_model_get_output_dtype", index)

    def _name(self, fn, index):
        s = ctypes.c_char_p()
        self._call(fn, self._h, index, ctypes.byref(s))
        return s.value.decode()

    def get_input_name(self, index):
        return self._name("ls_model_get_input_name", index)

    def get_output_name(self, index):
        return self._name("ls_model_get_output_name", index)

    def set_output_ptr(self, index, ptr):
        self._call("ls_model_set_output_ptr", self._h, index, _P(ptr))

    def get_output_ptr(self, index):
        p = _P()
        self._call("ls_model_get_output_ptr", self._h, index, ctypes.byref(p))
        return p.value

    def benchmark_mode(self, flag):
        self._call("ls_model_benchmark_mode", self._h, int(bool(flag)))

    def get_stream(self):
        p = _P()
        self._call("ls_model_get_stream", self._h, ctypes.byref(p))
        return p.value

    def set_profiling(self, on):
        self._call("ls_model_set_profiling", self._h, int(bool(on)))

    def get_profile(self):
        """Per-GEMM-site event timings accumulated since profiling was enabled."""
        import json
        buf = ctypes.create_string_buffer(8192)
        self._call("ls_model_get_profile", self._h, buf, 8192)
        return json.loads(buf.value.decode())

    def phase_times(self):
        """Generation models: (milliseconds before the step loop, milliseconds inside it, steps
        the loop ran) of the last ``Infer()``, between HIP events on the model's stream."""
        a, b, n = ctypes.c_float(0), ctypes.c_float(0), ctypes.c_int(0)
        self._call("ls_model_get_phase_times", self._h, ctypes.byref(a), ctypes.byref(b),
                   ctypes.byref(n))
        return a.value, b.value, n.value

    def graph_mode(self, flag):
        """QuantTransformer / QuantGpt: replay generation steps as HIP graphs."""
        self._call("ls_model_set_graph_mode", self._h, int(bool(flag)))

    def set_seed(self, seed):
        """QuantGpt with random sampling (topk > 1, topp): restart the generator states."""
        self._call("ls_model_set_seed", self._h, int(seed) & 0xFFFFFFFFFFFFFFFF)

    def graph_nodes(self):
        """Launches of one generation step: the nodes of the step graph captured last."""
        return self._int("ls_model_get_graph_nodes")

    def graph_stats(self):
        """(graphs captured, steps replayed) so far."""
        cap, rep = ctypes.c_int(0), ctypes.c_longlong(0)
        self._call("ls_model_get_graph_stats", self._h, ctypes.byref(cap), ctypes.byref(rep))
        return cap.value, rep.value

    def set_tap_step(self, step):
        """The generation step whose "dec.*" taps are copied (QuantTransformer, QuantGpt)."""
        self._call("ls_model_set_tap_step", self._h, int(step))

    def set_tap(self, layer, name, tensor):
        self._call("ls_model_set_tap", self._h, int(layer), name.encode(),
                   _P(None if tensor is None else tensor.data_ptr()))


class _HostIOModel(LSModel):
    """Adds the numpy-in / numpy-out behaviour of the reference's pybind classes."""

    def __init__(self, class_name, weight_path, max_batch_size):
        super().__init__(class_name, weight_path, max_batch_size)
        dev = torch.device("cuda:0")
        n_in = int(np.prod(self.get_input_max_shape(0)))
        self._d_input = torch.zeros(n_in, dtype=torch.int32, device=dev)
        self._d_outputs = []
        for i in range(self.get_output_size()):
            n_out = int(np.prod(self.get_output_max_shape(i)))
            t = torch.zeros(n_out, dtype=_TORCH_OF_DTYPE[self.get_output_dtype(i)], device=dev)
            self.set_output_ptr(i, t.data_ptr())
            self._d_outputs.append(t)
        torch.cuda.synchronize()

    def _upload(self, input_seq):
        a = np.ascontiguousarray(input_seq, dtype=np.int32)
        if a.ndim != 2:
            raise ValueError("input_seq must be a 2-D int32 array [batch, seq_len]")
        if a.size > self._d_input.numel():
            raise lib.LSHError(lib.LSH_ERR_INVALID, "input larger than the model's maximum shape",
                               "infer")
        self._d_input[:a.size].copy_(torch.from_numpy(a.reshape(-1)))
        torch.cuda.synchronize()
        self.set_input_ptr(0, self._d_input.data_ptr())
        self.set_input_shape(0, a.shape)
        return a.shape

    def _download(self, index):
        shape = self.get_output_shape(index)
        n = int(np.prod(shape))
        return self._d_outputs[index][:n].reshape(shape)


class QuantBert(_HostIOModel):
    """int8 BERT encoder: ``infer(token_ids) -> float32 [batch, seq_len, hidden]``."""

    def __init__(self, weight_path, max_batch_size):
        super().__init__("QuantBert", weight_path, max_batch_size)

    def infer(self, input_seq):
        self._upload(input_seq)
        self.infer_device()
        return self._download(0).float().cpu().numpy()

    def infer_fp16(self, input_seq):
        """Same as :meth:`infer` without the widening to float32."""
        self._upload(input_seq)
        self.infer_device()
        return self._download(0).cpu().numpy()


class QuantTransformer(_HostIOModel):
    """int8 encoder-decoder with beam search:
    ``infer(source_ids) -> (tokens int32 [batch, beam, out_len], scores float32 [batch, beam])``.
    """

    def __init__(self, weight_path, max_batch_size):
        super().__init__("QuantTransformer", weight_path, max_batch_size)

    def infer(self, input_seq):
        self._upload(input_seq)
        self.infer_device()
        return self._download(0).cpu().numpy(), self._download(1).cpu().numpy()

    def set_step_record(self, logits, alive_seq, max_steps):
        """Debug aid: device tensors that receive the per-step int8 logits
        [max_steps, batch*beam, vocab] and sequences [max_steps, batch*beam, max_step]."""
        self._call("ls_model_set_step_record", self._h,
                   _P(None if logits is None else logits.data_ptr()),
                   _P(None if alive_seq is None else alive_seq.data_ptr()), int(max_steps))

    def steps_run(self):
        return self._int("ls_model_get_steps_run")


class QuantGpt(_HostIOModel):
    """int8 GPT (wrapper.cc ``PyQuantGpt``): ``sample(token_ids) -> int32 [batch, sampled_len]``
    for model files with sampling_method "topk", ``ppl(token_ids) -> float32 [batch]`` for
    files with sampling_method "ppl"."""

    def __init__(self, weight_path, max_batch_size):
        super().__init__("QuantGpt", weight_path, max_batch_size)

    def infer(self, input_seq):
        self._upload(input_seq)
        self.infer_device()
        return self._download(0).cpu().numpy()

    sample = infer
    ppl = infer

    def set_step_record(self, logits, max_steps):
        """Debug aid: device tensor [max_steps, batch, vocab] int8 that receives the
        last-position logits of every sampling step."""
        self._call("ls_model_set_step_record", self._h,
                   _P(None if logits is None else logits.data_ptr()), _P(None), int(max_steps))

    def steps_run(self):
        return self._int("ls_model_get_steps_run")
