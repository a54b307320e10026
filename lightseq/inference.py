"""``lightseq.inference``: the three int8 model classes under the reference's module name
(lightseq/inference/pywrapper/wrapper.cc:944-976), so that scripts written as

    import lightseq.inference as lsi
    model = lsi.QuantBert("quant_bert.pb", 8)
    out = model.infer(token_ids)

run unchanged.  The float models of that module (Transformer, Gpt, Bert, Moe, Vit, T5 ...)
are not part of this build and raise on access with a message that says so.
"""
from lightseq_amd.inference import QuantBert, QuantGpt, QuantTransformer  # noqa: F401

__all__ = ["QuantBert", "QuantGpt", "QuantTransformer"]

_NOT_BUILT = ("Transformer", "Gpt", "Bert", "Moe", "Vit", "T5", "MT5", "XGLM", "QuantVit")


def __getattr__(name):
    if name in _NOT_BUILT:
        raise AttributeError(
            "lightseq.inference.%s: only the int8 models (QuantBert, QuantTransformer, QuantGpt) "
            "are provided by this MI355X build" % name)
    raise AttributeError("module 'lightseq.inference' has no attribute %r" % name)
