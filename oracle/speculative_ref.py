"""Acceptance of speculated (PARD) tokens and the rollback that follows, restated from
``Generator._postprocess_speculated_tokens`` (``pace/llm/generator.py:669-713``).
TEST INFRASTRUCTURE ONLY.

The reference handles batch 1 only (``generator.py:427-430``, and the hard-coded row 0
at ``:686-688``).  ``postprocess_row`` is that function for one row; a batch is the same
rule applied to every row on its own, which is what the product implements.

Pinning (``tests/test_host_logic.py``): the closed form "kept = 1 + longest common
prefix of the target's and the draft's first draft_size-1 tokens" by brute force over
every token combination of a small alphabet, and the removal count
``0 if all kept else draft_size - kept + 1`` (``:697-704``).
"""
from __future__ import annotations

from typing import List, Sequence, Tuple


def postprocess_row(next_tokens: Sequence[int], speculated_tokens: Sequence[int], draft_size: int) -> Tuple[List[int], int]:
    """(kept tokens, tokens to remove from the target model's cache) for one sequence.

    ``next_tokens``: the target model's ``draft_size`` tokens; ``speculated_tokens``: the
    draft's tokens, of which the last ``draft_size`` count (``:680``)."""
    spec = list(speculated_tokens)[-draft_size:]
    kept: List[int] = []
    for i in range(draft_size - 1):          # the last position is the target's own token (:683-690)
        if next_tokens[i] == spec[i]:
            kept.append(int(next_tokens[i]))
        else:
            break
    kept.append(int(next_tokens[len(kept)]))  # the token the target model generated (:693)
    removed = draft_size - len(kept)
    # +1: the token fed again at the start of the next iteration (:697-704)
    return kept, (removed + 1 if removed > 0 else 0)
