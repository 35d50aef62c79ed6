"""Loading the reference's checkpoints into m2_amd modules.

The reference loads Composer checkpoints with `from_composer` (bert/src/bert_layers.py:1087-1209): the weights sit
under `state['model']`, the keys carry a `model.` prefix from the Composer wrapper and, below it, `bert.` for the
encoder inside the task model; when a short-context checkpoint is extended to a longer context the position
embedding table is repeated, `position_ids` and the filters' `pos_emb.t` are dropped (the longer model keeps its
own) and `pos_emb.z` is extended (:1122-1168, and `expand_8k_model_to_32k`,
bert/src/embeddings/training_functions.py:430-472).

Files are read with `torch.load(..., weights_only=True)`: nothing in a checkpoint is executed.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional, Tuple, Union

import torch
import torch.nn as nn

PREFIXES = ("model.", "bert.")


def unwrap_state_dict(obj: Mapping) -> Dict[str, torch.Tensor]:
    """The tensor dict inside a checkpoint object: Composer's `{'state': {'model': ...}}`, a `{'model': ...}` or
    `{'state_dict': ...}` wrapper, or a plain state dict."""
    if "state" in obj and isinstance(obj["state"], Mapping) and "model" in obj["state"]:
        obj = obj["state"]["model"]
    elif "model" in obj and isinstance(obj["model"], Mapping):
        obj = obj["model"]
    elif "state_dict" in obj and isinstance(obj["state_dict"], Mapping):
        obj = obj["state_dict"]
    bad = [k for k, v in obj.items() if not isinstance(v, torch.Tensor)]
    if bad:
        raise ValueError(f"not a state dict: entries {bad[:3]} are not tensors")
    return dict(obj)


def strip_prefixes(sd: Mapping[str, torch.Tensor], prefixes=PREFIXES) -> Tuple[Dict[str, torch.Tensor], List[str]]:
    """Removes `model.` and then `bert.` from the keys that carry them (consume_prefix_in_state_dict_if_present,
    bert_layers.py:1190, plus the `.bert` attribute the reference takes, embeddings_inference.py:247).  Keys of the
    task heads around the encoder (`cls.*`, `classifier.*`, `dropout.*`) are returned separately."""
    out, heads = {}, []
    for k, v in sd.items():
        k2 = k
        if k2.startswith("model."):
            k2 = k2[len("model."):]
        if k2.startswith("bert."):
            k2 = k2[len("bert."):]
        elif k2.split(".")[0] in ("cls", "classifier", "dropout", "qa_outputs"):
            heads.append(k)
            continue
        out[k2] = v
    return out, heads


# slots of the zero tensor that receive the old pos_emb.z table in the reference's expansion, by old context length:
# `for k in range(2, R): z_new[(k - 1) * L_old : k * L_old] = z_old` with R = {1024: 3, 128: 17, 4096: 11, 8192: 5}
# (bert/src/bert_layers.py:1141-1151, bert/src/embeddings/training_functions.py:452-460), i.e. slots 1 .. R - 2
REFERENCE_Z_SLOTS = {1024: 1, 128: 15, 4096: 9, 8192: 3}


def extend_context(sd: Mapping[str, torch.Tensor], new_len: int, tile_pos_emb_z: bool = False, mode: Optional[str] = None,
                   z_slots: Optional[int] = None) -> Dict[str, torch.Tensor]:
    """A state dict trained at context L_old, prepared for a model built for `new_len` = r * L_old tokens:

    * `embeddings.position_embeddings.weight` (L_old, d) is repeated r times (bert_layers.py:1122-1131);
    * `embeddings.position_ids` and every `pos_emb.t` are dropped: the longer model keeps the ones it builds for
      its own length (:1137, :1159-1161);
    * every `pos_emb.z` (1, L_old, emb), according to `mode`:
        "reference"  what the reference does (:1141-1151): a ZERO tensor of the new length with the old table
                     written into slots 1 .. n (slot j = positions [j L_old, (j + 1) L_old)); slot 0 and the slots
                     after n stay zero.  n = `z_slots`, else the reference's own count for that L_old
                     (REFERENCE_Z_SLOTS: 3 for 8192 -> 32768, 15 for 128 -> 2048), else every slot but the first;
                     slots that do not fit the new length are left out.  (The reference allocates 16 L_old
                     positions whatever the target; here the tensor has the new model's length.)
        "closed_form" (default)  dropped, so that the longer model keeps the closed-form embedding of its own
                     length (bert/src/mm/hyena_utils.py:66-88);
        "tile"       repeated r times along the sequence (also selected by tile_pos_emb_z=True).
    A checkpoint that was fine-tuned after the reference's expansion carries filters trained against the
    "reference" table: use that mode to reproduce its filters.
    """
    if mode is None:
        mode = "tile" if tile_pos_emb_z else "closed_form"
    if mode not in ("reference", "closed_form", "tile"):
        raise ValueError(f"unknown pos_emb.z extension mode {mode!r}")
    out = dict(sd)
    key = "embeddings.position_embeddings.weight"
    if key in out:
        old = out[key].shape[0]
        if new_len % old != 0:
            raise ValueError(f"cannot extend a context of {old} to {new_len}: not a multiple")
        out[key] = out[key].repeat(new_len // old, 1)
    out.pop("embeddings.position_ids", None)
    for k in list(out):
        if k.endswith("pos_emb.t"):
            del out[k]
        elif k.endswith("pos_emb.z"):
            z = out.pop(k)
            old = z.shape[1]
            if mode == "closed_form":
                continue
            if new_len % old != 0:
                raise ValueError(f"{k}: cannot extend {old} positions to {new_len}: not a multiple")
            if mode == "tile":
                out[k] = z.repeat(1, new_len // old, 1)
            else:
                n = z_slots if z_slots is not None else REFERENCE_Z_SLOTS.get(old, new_len // old - 1)
                znew = torch.zeros(z.shape[0], new_len, z.shape[2], dtype=z.dtype)
                for slot in range(1, n + 1):
                    if (slot + 1) * old <= new_len:
                        znew[:, slot * old:(slot + 1) * old, :] = z
                out[k] = znew
    return out


def load_reference_checkpoint(model: nn.Module, checkpoint: Union[str, Mapping], extend_to: Optional[int] = None,
                              tile_pos_emb_z: bool = False, max_missing: int = 5,
                              z_mode: Optional[str] = None) -> Tuple[List[str], List[str]]:
    """Loads a reference checkpoint (a path, or an already loaded object) into `model` (an m2_amd BertModel, or any
    module with the same key names).  Returns (missing_keys, unexpected_keys) like `load_state_dict(strict=False)`;
    `z_mode` picks how `pos_emb.z` is lengthened (see `extend_context`; "reference" reproduces the reference's zero-filled
    expansion).  Raises if more than `max_missing` keys of the model are absent (the reference's own sanity threshold,
    embeddings_inference.py:244-246) or if a tensor has the wrong shape."""
    obj = torch.load(checkpoint, map_location="cpu", weights_only=True) if isinstance(checkpoint, str) else checkpoint
    sd, heads = strip_prefixes(unwrap_state_dict(obj))
    if extend_to is not None:
        sd = extend_context(sd, extend_to, tile_pos_emb_z, mode=z_mode)
    own = model.state_dict()
    for k, v in sd.items():
        if k in own and tuple(own[k].shape) != tuple(v.shape):
            raise ValueError(f"{k}: checkpoint has shape {tuple(v.shape)}, the model expects {tuple(own[k].shape)}"
                             + (" (pass extend_to= to lengthen the context)" if "pos" in k else ""))
    missing, unexpected = model.load_state_dict(sd, strict=False)
    missing, unexpected = list(missing), list(unexpected) + heads
    if len(missing) > max_missing:
        raise RuntimeError(f"{len(missing)} keys of the model are not in the checkpoint, e.g. {missing[:5]}")
    if hasattr(model, "encoder") and hasattr(model.encoder, "reset_graphs"):
        model.encoder.reset_graphs()
    return missing, unexpected
