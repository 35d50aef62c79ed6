"""m2_amd: MI355X (gfx950) kernels for the forward hot path of M2-BERT's Monarch Mixer, behind the
reference's PyTorch module surface.  Importing the package loads libm2_amd.so and fails if it has
not been built (`python m2_amd/build.py`); nothing here runs on the CPU."""
from .config import M2BertConfig, m2_bert_80m, m2_bert_110m, m2_bert_341m, m2_bert_large
from .init import seeded_state_dict
from . import ops
from .hyena import HyenaFilter, Sin, PositionalEmbedding, ExponentialModulation
from .mixer import MonarchMixerSequenceMixing
from .blockdiag import BlockdiagLinear, blockdiag_multiply
from .encoder import BertEmbeddings, BertGatedLinearUnitMLP, BertLayer, BertEncoder, BertModel, BertPooler
from .embed import M2BertTextEncoder
from .checkpoint import load_reference_checkpoint, extend_context

__all__ = ["M2BertConfig", "m2_bert_80m", "m2_bert_110m", "m2_bert_341m", "m2_bert_large", "seeded_state_dict", "ops", "HyenaFilter", "Sin",
           "PositionalEmbedding", "ExponentialModulation", "MonarchMixerSequenceMixing", "BlockdiagLinear",
           "blockdiag_multiply", "BertEmbeddings", "BertGatedLinearUnitMLP", "BertLayer", "BertEncoder", "BertModel",
           "BertPooler", "M2BertTextEncoder", "load_reference_checkpoint", "extend_context"]
