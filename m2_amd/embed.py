"""Embedding-inference caller: batches of texts -> pooled embeddings, the loop of the reference's
`M2_BERT_Encoder.encode_queries` / `encode_corpus` (bert/embeddings_inference.py:267-351).

The reference tokenises with a Hugging Face tokenizer it downloads; here the tokenizer is whatever
callable the caller passes (`tokenizer([text], return_tensors="pt")` -> mapping with `input_ids` and
`attention_mask` of shape (1, n), which is the Hugging Face calling convention), or the caller passes
token ids directly to `encode_token_ids`.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Optional, Sequence

import numpy as np
import torch
import torch.nn.functional as F

from .encoder import BertModel


def split_list(items: Sequence, chunk_size: int) -> Iterable[Sequence]:
    """Consecutive chunks of at most chunk_size items (bert/embeddings_inference.py:60-62)."""
    for i in range(0, len(items), chunk_size):
        yield items[i:i + chunk_size]


def pad_or_truncate(ids: torch.Tensor, length: int) -> torch.Tensor:
    """(1, n) -> (1, length): zero padding on the right, or truncation (`expand_tensor` followed by the slice,
    bert/embeddings_inference.py:38-43,278-283)."""
    if ids.shape[1] < length:
        ids = F.pad(ids, [0, length - ids.shape[1]])
    return ids[:, :length]


class M2BertTextEncoder:
    """`model`: a BertModel with a pooler, on the GPU, in eval mode.  Every text is padded or cut to
    `max_seq_len` tokens (the reference's `evaluation_max_seq_len`), texts are run `batch_size` at a time and the
    pooled outputs are collected on the host."""

    def __init__(self, model: BertModel, max_seq_len: int, tokenizer: Optional[Callable] = None,
                 device: Optional[torch.device] = None):
        if model.pooler is None:
            raise ValueError("the embedding caller needs a BertModel built with add_pooling_layer=True")
        self.model = model.eval()
        self.max_seq_len = int(max_seq_len)
        self.tokenizer = tokenizer
        self.device = device if device is not None else next(model.parameters()).device

    # -- the loop ----------------------------------------------------------------------------------
    def encode_token_ids(self, token_ids: Sequence, batch_size: int,
                         attention_masks: Optional[Sequence] = None) -> np.ndarray:
        """token_ids: one 1-D sequence of ids per text (any lengths, may be empty); returns (len(token_ids), d)
        fp32.  Without attention_masks every given token counts as real and the padding as masked."""
        out = torch.empty(0, self.model.config.hidden_size)
        for lo in range(0, len(token_ids), batch_size):
            ids_rows, mask_rows = [], []
            for k in range(lo, min(lo + batch_size, len(token_ids))):
                ids = torch.as_tensor(token_ids[k], dtype=torch.long).reshape(1, -1)
                mask = torch.ones_like(ids) if attention_masks is None else \
                    torch.as_tensor(attention_masks[k], dtype=torch.long).reshape(1, -1)
                if mask.shape != ids.shape:
                    raise ValueError(f"text {k}: {ids.shape[1]} token ids but {mask.shape[1]} mask entries")
                ids_rows.append(pad_or_truncate(ids, self.max_seq_len))
                mask_rows.append(pad_or_truncate(mask, self.max_seq_len))
            ids_b = torch.cat(ids_rows, 0).to(self.device)
            mask_b = torch.cat(mask_rows, 0).to(self.device)
            with torch.no_grad():
                _, pooled = self.model(input_ids=ids_b, attention_mask=mask_b)
            out = torch.cat((out, pooled.detach().float().cpu()), 0)
        if torch.isnan(out).any():
            raise ValueError("NaNs in the encoded texts")
        return out.numpy()

    def _encode_texts(self, texts: List[str], batch_size: int) -> np.ndarray:
        if self.tokenizer is None:
            raise ValueError("no tokenizer was given: use encode_token_ids, or pass tokenizer= to the constructor")
        ids, masks = [], []
        for text in texts:
            enc = self.tokenizer([text], return_tensors="pt")
            ids.append(enc["input_ids"].reshape(-1))
            masks.append(enc["attention_mask"].reshape(-1))
        return self.encode_token_ids(ids, batch_size, attention_masks=masks)

    # -- the reference's two entry points ------------------------------------------------------------
    def encode_queries(self, queries: List[str], batch_size: int, **kwargs) -> np.ndarray:
        return self._encode_texts(list(queries), batch_size)

    def encode_corpus(self, corpus: List[Dict[str, str]], batch_size: int, **kwargs) -> np.ndarray:
        """Passages are dicts with 'title' and 'text'; the title is prepended when the model reads at least
        512 tokens (bert/embeddings_inference.py:316-319)."""
        if self.max_seq_len >= 512:
            texts = [p["title"] + " " + p["text"] for p in corpus]
        else:
            texts = [p["text"] for p in corpus]
        return self._encode_texts(texts, batch_size)
