"""Configuration of the M2-BERT encoder, field names as the reference reads them.

The reference merges a YAML `model_config` into a Hugging Face `BertConfig`
(bert/src/create_bert.py:85-92, bert/src/configuration_bert.py:4-78); the fields that exist only
through the YAML (`long_conv_l_max`, `hyena_w`, `hyena_emb_dim` ... read at
bert/src/bert_layers.py:530-538) are ordinary fields here.  Defaults are the 80M pre-training
recipe (bert/yamls/pretrain/monarch-mixer-pretrain-786dim-80m-parameters.yaml:17-38) on top of
`bert-base-uncased` (hidden 768, 12 layers, intermediate 3072, eps 1e-12, vocab 30522 padded to a
multiple of 8 = 30528).
"""
from __future__ import annotations

from dataclasses import dataclass, replace


@dataclass
class M2BertConfig:
    # bert-base-uncased
    vocab_size: int = 30528
    hidden_size: int = 768
    num_hidden_layers: int = 12
    num_attention_heads: int = 12
    intermediate_size: int = 3072
    hidden_dropout_prob: float = 0.1
    attention_probs_dropout_prob: float = 0.0
    max_position_embeddings: int = 128
    type_vocab_size: int = 2
    layer_norm_eps: float = 1e-12
    pad_token_id: int = 0
    initializer_range: float = 0.02
    # Monarch Mixer
    monarch_mixer_sequence_mixing: bool = True
    long_conv_l_max: int = 128
    long_conv_kernel_learning_rate: float = 1e-3
    hyena_lr_pos_emb: float = 1e-5
    hyena_w: int = 10
    hyena_w_mod: int = 1
    hyena_wd: float = 0.1
    hyena_emb_dim: int = 5
    hyena_filter_dropout: float = 0.2
    hyena_filter_order: int = 128
    hyena_training_additions: bool = False
    bidirectional: bool = True
    residual_long_conv: bool = True
    use_glu_mlp: bool = True
    use_monarch_mlp: bool = True
    monarch_mlp_nblocks: int = 4
    use_positional_encodings: bool = True
    use_flash_mm: bool = False
    use_flash_fft: bool = False
    pool_all: bool = False                     # BertPooler: masked mean over the sequence instead of the first token
    use_cls_token: bool = False                # read by the reference's pooler constructor, not by its forward
    sequence_token_planting: bool = False
    attention_pooling: bool = False

    def with_seq_len(self, L: int) -> "M2BertConfig":
        return replace(self, max_position_embeddings=L, long_conv_l_max=L)


def m2_bert_80m(seq_len: int = 128) -> M2BertConfig:
    return M2BertConfig().with_seq_len(seq_len)


def m2_bert_large(seq_len: int = 128, num_hidden_layers: int = 24) -> M2BertConfig:
    """d_model 1536 / intermediate 6144 (bert/yamls/pretrain/monarch-mixer-large-pretrain-1536dim-260m-parameters.yaml)."""
    return replace(M2BertConfig(), hidden_size=1536, intermediate_size=6144, num_hidden_layers=num_hidden_layers,
                   num_attention_heads=24).with_seq_len(seq_len)


def m2_bert_110m(seq_len: int = 128) -> M2BertConfig:
    """d_model 960 / intermediate 3840, 12 layers: the parameter-matched model
    (bert/yamls/pretrain/monarch-mixer-pretrain-960dim-parameter-matched.yaml:17-24).  Its MLP blocks are 240 wide."""
    return replace(M2BertConfig(), hidden_size=960, intermediate_size=3840).with_seq_len(seq_len)


def m2_bert_341m(seq_len: int = 128) -> M2BertConfig:
    """d_model 1792 / intermediate 7168, 12 layers
    (bert/yamls/pretrain/monarch-mixer-large-pretrain-1792dim-341m-parameters.yaml:17-24)."""
    return replace(M2BertConfig(), hidden_size=1792, intermediate_size=7168).with_seq_len(seq_len)
