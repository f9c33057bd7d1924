"""Ragged speculative-decoding glue: which draft tokens each sequence keeps and how far each
sequence's KV cache rolls back.

The reference implements this for one sequence (``Generator._postprocess_speculated_tokens``,
``pace/llm/generator.py:669-713``; batch > 1 is refused at ``:427-430``) because its caches
hold one length for the whole batch.  The paged cache keeps a length per sequence, so the same
rule is applied row by row and the rollback is a per-sequence ``truncate``.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np
import torch


def accepted_counts(next_tokens: torch.Tensor, speculated_tokens: torch.Tensor, draft_size: int) -> np.ndarray:
    """Tokens kept per sequence: the matching prefix of the first ``draft_size - 1`` positions
    plus the target model's own next token (``generator.py:683-693``).  ``next_tokens`` is
    ``[B, draft_size]``, ``speculated_tokens`` ``[B, >= draft_size]`` (its tail counts, ``:680``)."""
    spec = speculated_tokens[:, -draft_size:]
    if next_tokens.shape[1] != draft_size or spec.shape != next_tokens.shape:
        raise ValueError(f"expected [B, {draft_size}] token ids, got {tuple(next_tokens.shape)} and {tuple(spec.shape)}")
    same = (next_tokens[:, : draft_size - 1] == spec[:, : draft_size - 1]).to(torch.int64)
    prefix = torch.cumprod(same, dim=1).sum(dim=1)  # length of the leading run of matches
    return (prefix + 1).cpu().numpy().astype(np.int64)


def kept_tokens(next_tokens: torch.Tensor, counts: np.ndarray) -> List[torch.Tensor]:
    """The accepted ids of every sequence (ragged: ``counts[b]`` each)."""
    return [next_tokens[b, : int(c)] for b, c in enumerate(counts)]


def rollback_lengths(counts: np.ndarray, draft_size: int) -> np.ndarray:
    """Tokens to drop from each sequence of the target model's cache: nothing where every draft
    was accepted, else the rejected ones plus the token that is fed again (``generator.py:697-704``)."""
    removed = draft_size - np.asarray(counts, dtype=np.int64)
    if (removed < 0).any():
        raise ValueError("a sequence cannot keep more tokens than were drafted")
    return np.where(removed > 0, removed + 1, 0)


def rollback(cache_manager, counts: np.ndarray, draft_size: int) -> np.ndarray:
    """Apply ``rollback_lengths`` to every layer of a paged ``KVCacheManager``; returns them."""
    drop = rollback_lengths(counts, draft_size)
    if drop.any():
        for layer in cache_manager.cache_objects:
            layer.truncate(drop)
    return drop


def right_aligned(rows: Sequence[torch.Tensor], width: int, pad_value=0) -> Tuple[torch.Tensor, np.ndarray]:
    """Stack ragged per-sequence rows ``[n_b, ...]`` into ``[B, width, ...]``, each sequence's rows at
    the end.  The multi-token attention entry point gives row ``s`` of sequence ``b`` the tokens
    ``<= len_b - width + s``, so with this alignment the last ``n_b`` rows are exactly the causal
    rows of the sequence's ``n_b`` new tokens; the leading rows are padding to ignore.
    Returns the stacked tensor and the counts."""
    counts = np.asarray([int(r.shape[0]) for r in rows], dtype=np.int64)
    if counts.max(initial=0) > width:
        raise ValueError(f"a sequence has {int(counts.max())} rows, more than the width {width}")
    first = rows[0]
    out = first.new_full((len(rows), width) + tuple(first.shape[1:]), pad_value)
    for b, r in enumerate(rows):
        if r.shape[0]:
            out[b, width - r.shape[0]:] = r
    return out, counts
