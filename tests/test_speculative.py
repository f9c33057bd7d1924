"""Ragged speculative-decoding glue: acceptance rule and rollback arithmetic against the
restatement of the reference's batch-1 function (CPU), and a ragged verify loop on the GPU."""
import itertools

import numpy as np
import pytest
import torch

from helpers import assert_attention_close, assert_bits_equal, seeded_kv, seeded_q
from oracle.paged_ref import RaggedCacheModel
from oracle.speculative_ref import postprocess_row
from pace_mi355.llm import speculative


def test_oracle_row_rule_is_the_longest_common_prefix_plus_one():
    """Brute force over every pair of length-3 strings on a 2-letter alphabet."""
    d = 3
    for nxt in itertools.product([7, 9], repeat=d):
        for spec in itertools.product([7, 9], repeat=d):
            kept, removed = postprocess_row(nxt, spec, d)
            lcp = 0
            while lcp < d - 1 and nxt[lcp] == spec[lcp]:
                lcp += 1
            assert kept == list(nxt[: lcp + 1])
            assert removed == (0 if lcp + 1 == d else d - (lcp + 1) + 1)
    # only the last draft_size speculated ids count (generator.py:680)
    assert postprocess_row([1, 2, 3], [99, 98, 1, 2, 5], 3) == ([1, 2, 3], 0)


@pytest.mark.parametrize("draft_size", [1, 2, 4, 8])
def test_batched_counts_equal_the_reference_rule_row_by_row(draft_size):
    g = torch.Generator().manual_seed(draft_size)
    B = 64
    nxt = torch.randint(0, 3, (B, draft_size), generator=g)
    spec = torch.randint(0, 3, (B, draft_size + 2), generator=g)
    spec[:8, -draft_size:] = nxt[:8]  # some rows accept everything
    counts = speculative.accepted_counts(nxt, spec, draft_size)
    drop = speculative.rollback_lengths(counts, draft_size)
    kept = speculative.kept_tokens(nxt, counts)
    for b in range(B):
        want_kept, want_drop = postprocess_row(nxt[b].tolist(), spec[b].tolist(), draft_size)
        assert kept[b].tolist() == want_kept and int(drop[b]) == want_drop
    assert (counts[:8] == draft_size).all() and (drop[:8] == 0).all()
    with pytest.raises(ValueError):
        speculative.accepted_counts(nxt[:, :-1] if draft_size > 1 else nxt[:, :0], spec, draft_size)
    with pytest.raises(ValueError):
        speculative.rollback_lengths(np.array([draft_size + 1]), draft_size)


def test_right_aligned_padding():
    rows = [torch.arange(6).view(3, 2), torch.zeros(0, 2, dtype=torch.long), torch.arange(2).view(1, 2)]
    out, counts = speculative.right_aligned(rows, 4, pad_value=-1)
    assert counts.tolist() == [3, 0, 1] and out.shape == (3, 4, 2)
    assert out[0, 1:].tolist() == rows[0].tolist() and (out[0, 0] == -1).all()
    assert (out[1] == -1).all() and out[2, 3].tolist() == [0, 1]
    with pytest.raises(ValueError):
        speculative.right_aligned(rows, 2)


@pytest.mark.gpu
def test_ragged_verify_loop_batch_of_three(device):
    """Two verify iterations with a different number of new tokens per sequence and a different
    rollback per sequence -- the case the reference cannot run (generator.py:427-430)."""
    from pace_mi355.llm import KVCacheManager, KVCacheType

    class Cfg:
        num_hidden_layers = 2
        num_attention_heads = 8
        num_key_value_heads = 2

    B, hkv, n_rep, D, draft = 3, 2, 4, 128, 4
    mgr = KVCacheManager(Cfg(), 160, KVCacheType.PAGED)
    models = [RaggedCacheModel(B, hkv, D) for _ in range(2)]
    prompt = [20, 33, 7]
    for layer in range(2):
        k, v = seeded_kv(10 + layer, B, hkv, max(prompt), D)
        mgr[layer].append_ragged(k.to(device), v.to(device), prompt)
        models[layer].append(k, v, prompt)
    new_counts = [[4, 4, 4], [2, 4, 1], [4, 3, 3]]  # tokens each sequence feeds per iteration
    accepted = [np.array([1, 4, 3]), np.array([2, 2, 1]), np.array([4, 1, 2])]
    for it, counts in enumerate(new_counts):
        W = max(counts)
        for layer in range(2):
            rows_k, rows_v, rows_q = [], [], []
            for b, c in enumerate(counts):
                k, v = seeded_kv(100 * it + 10 * layer + b, 1, hkv, c, D)
                rows_k.append(k[0].transpose(0, 1)), rows_v.append(v[0].transpose(0, 1))  # [c, H, D]
                rows_q.append(seeded_q(500 + 100 * it + 10 * layer + b, 1, hkv * n_rep, c, D)[0].transpose(0, 1))
            kp, _ = speculative.right_aligned(rows_k, W)
            vp, _ = speculative.right_aligned(rows_v, W)
            qp, _ = speculative.right_aligned(rows_q, W)
            kp, vp, qp = (t.transpose(1, 2).contiguous() for t in (kp, vp, qp))  # [B, H, W, D]
            mgr[layer].append_ragged(kp.to(device), vp.to(device), counts, right_aligned=True)
            # the oracle model takes left-aligned rows
            kl = torch.zeros_like(kp)
            vl = torch.zeros_like(vp)
            for b, c in enumerate(counts):
                kl[b, :, :c], vl[b, :, :c] = kp[b, :, W - c:], vp[b, :, W - c:]
            models[layer].append(kl, vl, counts)
            out = mgr[layer].attend(qp.to(device))
            want = models[layer].attention(qp, n_rep)
            for b, c in enumerate(counts):
                assert_attention_close(out[b, :, W - c:], want[b, :, W - c:], f"iteration {it} layer {layer} sequence {b}")
        keep = np.minimum(accepted[it], np.array(counts))
        drop = np.where(np.array(counts) - keep > 0, np.array(counts) - keep + 1, 0)
        drop = np.minimum(drop, np.array(counts))
        for layer in range(2):
            mgr[layer].truncate(drop)
            models[layer].truncate(drop.tolist())
            K, V = models[layer].dense()
            gk, gv = mgr[layer].gather(n_rep=1)
            assert_bits_equal(gk, K, f"K after rollback {it} layer {layer}")
            assert_bits_equal(gv, V, f"V after rollback {it} layer {layer}")
    assert len(mgr) == max(models[0].seq_lens())


@pytest.mark.gpu
def test_rollback_helper_truncates_every_layer(device):
    from pace_mi355.llm import KVCacheManager, KVCacheType

    class Cfg:
        num_hidden_layers = 3
        num_attention_heads = 4
        num_key_value_heads = 4

    mgr = KVCacheManager(Cfg(), 64, KVCacheType.PAGED)
    for layer in range(3):
        k, v = seeded_kv(layer, 2, 4, 30, 64)
        mgr[layer].update_cache(k.to(device), v.to(device), 2)
    drop = speculative.rollback(mgr, np.array([4, 2]), 4)
    assert drop.tolist() == [0, 3]
    for layer in range(3):
        assert mgr[layer].lens.tolist() == [30, 27]
