"""Drop-in module name of the reference's Python package for the int8 inference path.

``import lightseq.inference as lsi`` gives ``lsi.QuantBert``, ``lsi.QuantTransformer`` and
``lsi.QuantGpt`` with the constructor and methods that the reference's pybind module
registers (lightseq/inference/pywrapper/wrapper.cc:944-976), implemented by
``lightseq_amd`` on MI355X.  Nothing else of the reference's package is provided.
"""
__version__ = "3.0.1"
