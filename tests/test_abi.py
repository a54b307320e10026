"""The C-ABI library loads and exports every symbol that include/*.h declares, and
the ctypes signature table of the Python host matches the header prototypes.
No GPU work is launched here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("lightseq_hip.h", "lightseq_ops.h", "lightseq_model.h")]
PROTO_RE = re.compile(r"^\s*(?:const\s+char\s*\*|int|float)\s+((?:lsh|ls)_\w+)\s*\(([^;]*?)\)\s*;",
                      re.M | re.S)


def _prototypes():
    out = {}
    for h in HEADERS:
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        for name, args in PROTO_RE.findall(text):
            out[name] = " ".join(args.split())
    return out


def _code(arg):
    arg = arg.strip()
    if arg == "void":
        return ""
    if re.match(r"const\s+char\s*\*", arg):
        return "c"
    if "*" in arg:
        return "p"
    if arg.startswith("lsh_stream_t"):
        return "s"
    if arg.startswith("float"):
        return "f"
    if arg.startswith("int64_t"):
        return "l"
    if arg.startswith("uint64_t") or arg.startswith("unsigned long long"):
        return "Q"
    if arg.startswith("int"):
        return "i"
    raise AssertionError("unhandled parameter type: %r" % arg)


def test_header_declares_something():
    protos = _prototypes()
    assert len(protos) > 50
    assert "lsh_gemm_i8_i8o" in protos and "ls_model_create" in protos


def test_library_exports_every_declared_symbol():
    from lightseq_amd import lib
    L = lib.load()
    missing = [n for n in _prototypes() if not hasattr(L, n)]
    assert not missing, missing
    assert lib.version().startswith("lightseq_hip")
    assert lib.last_error() == ""


def test_ctypes_table_matches_header():
    from lightseq_amd import lib
    protos = _prototypes()
    for name, (typed, codes) in lib._SIGNATURES.items():
        for suffix in (("_f16", "_f32") if typed else ("",)):
            full = name + suffix
            assert full in protos, full
            want = "".join(_code(a) for a in protos[full].split(","))
            assert want == codes, (full, want, codes)
    # and nothing in lightseq_hip.h / lightseq_ops.h is left unbound
    bound = {n + s for n, (t, _) in lib._SIGNATURES.items() for s in (("_f16", "_f32") if t else ("",))}
    kernels_header = re.sub(r"/\*.*?\*/", "", open(HEADERS[0]).read() + open(HEADERS[1]).read(),
                            flags=re.S)
    declared = {n for n, _ in PROTO_RE.findall(kernels_header)} - {"lsh_last_error", "lsh_version",
                                                                         "lsh_length_norm"}
    assert declared == bound, declared ^ bound


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from lightseq_amd import lib
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        lib.load()


def test_status_codes_without_gpu():
    """Argument validation happens before any launch, so it is testable on the CPU."""
    from lightseq_amd import lib
    L = lib.load()
    rc = L.lsh_launch_quantize_tensor_f16(None, None, 1, 8, ctypes.c_float(1.0), None, 1)
    assert rc == lib.LSH_ERR_UNSUPPORTED and "COL32" in lib.last_error()
    rc = L.lsh_gemm_i8_i32o(None, None, None, 4, 4, 16, None)
    assert rc == lib.LSH_ERR_INVALID
    rc = L.lsh_launch_enc_emb_i8I_f16(None, None, None, None, None, 0, 1, 1, 8, None, None, None, 1,
                                      ctypes.c_float(1.0), 0)
    assert rc == lib.LSH_ERR_INVALID and "multilingle" in lib.last_error()


def test_reference_module_name_exposes_the_int8_models():
    """`import lightseq.inference as lsi` is what the reference's users write
    (lightseq/inference/pywrapper/wrapper.cc:944-976 registers the classes there)."""
    import lightseq.inference as lsi
    from lightseq_amd import inference
    assert lsi.QuantBert is inference.QuantBert
    assert lsi.QuantTransformer is inference.QuantTransformer
    assert lsi.QuantGpt is inference.QuantGpt
    for method in ("infer",):
        assert callable(getattr(lsi.QuantBert, method)) and callable(getattr(lsi.QuantTransformer, method))
    assert callable(lsi.QuantGpt.sample) and callable(lsi.QuantGpt.ppl)
    with pytest.raises(AttributeError, match="only the int8 models"):
        lsi.Bert
