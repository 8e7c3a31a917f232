"""Logits of the plain implementation for a model folder and a token list, computed once."""
import numpy as np
import torch

from .plain import model as plain_model

_folders = {}
_logits = {}


def plain_logits(folder, tokens):
    """float32 array [len(tokens), vocab] from the plain whole-sequence forward pass."""
    key = (folder, tuple(tokens))
    if key not in _logits:
        if folder not in _folders:
            _folders[folder] = plain_model.read_folder(folder, torch.float32)
        cfg, w = _folders[folder]
        _logits[key] = plain_model.forward(cfg, w, list(tokens)).numpy().astype(np.float32)
    return _logits[key]


def plain_rows(folder, tokens, rows):
    """{position: float32 logits [vocab]} at `rows` only (for models whose vocabulary makes every
    position's logits too much to keep)."""
    rows = sorted(set(rows))
    key = (folder, tuple(tokens), tuple(rows))
    if key not in _logits:
        if folder not in _folders:
            _folders[folder] = plain_model.read_folder(folder, torch.float32)
        cfg, w = _folders[folder]
        _logits[key] = plain_model.forward(cfg, w, list(tokens), rows=rows).numpy().astype(np.float32)
    out = _logits[key]
    return {p: out[i] for i, p in enumerate(rows)}


def forget(folder):
    """Drop a folder's weights and logits (large models)."""
    _folders.pop(folder, None)
    for key in [k for k in _logits if k[0] == folder]:
        del _logits[key]


def plain_folder(folder):
    if folder not in _folders:
        _folders[folder] = plain_model.read_folder(folder, torch.float32)
    return _folders[folder]
