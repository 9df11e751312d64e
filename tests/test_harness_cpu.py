"""Host-side pieces of the check-and-benchmark matrix (flash_mi355/harness.py)."""
import numpy as np
import torch

from flash_mi355 import harness as Hn
from oracle import attention_oracle as O


def test_flop_convention_matches_reference_formula():
    # testing.py:92-107: 4*B*H*L*L*D, halved when causal; backward 2.0x for eager, 2.5x for fused
    shape = [2, 4, 256, 64]
    dense = 4.0 * 2 * 4 * 256 * 256 * 64
    assert Hn.attention_flops(shape, False, "fwd", "mi355") == dense
    assert Hn.attention_flops(shape, True, "fwd", "mi355") == dense / 2
    assert Hn.attention_flops(shape, True, "bwd", "torch") == dense
    assert Hn.attention_flops(shape, True, "bwd", "mi355") == dense * 1.25
    assert Hn.attention_flops(shape, False, "fb", "math") == dense * 3
    assert Hn.attention_flops(shape, False, "fb", "mem") == dense * 3.5


def test_sampled_ids_and_mask_agree_with_the_oracle_mask():
    torch.manual_seed(3)
    shape = [2, 3, 96, 16]
    for causal in (False, True):
        eq, ek, keep = Hn.sample_doc_ids(shape, "cpu", causal)
        assert eq.shape == (2, 3, 96) and keep.shape == (2, 1, 96, 96)
        assert (eq[:, 0] == eq[:, 2]).all()
        ids = eq[:, 0].numpy()
        assert (np.diff(ids, axis=1) >= 0).all() and (ids < 0).any() and (ids >= 0).any()
        ref = O.keep_mask(96, 96, causal, eq.numpy(), ek.numpy(), 1)
        assert np.array_equal(np.broadcast_to(keep.numpy(), ref.shape), ref)


def test_eager_comparator_is_the_closed_form():
    torch.manual_seed(4)
    q, k, v = (torch.randn(1, 2, 40, 16) for _ in range(3))
    _, _, keep = Hn.sample_doc_ids([1, 2, 40, 16], "cpu", True)
    got = Hn.attn_torch(q, k, v, False, attn_mask=keep)
    eq, ek, _ = (None, None, None)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=keep)
    assert torch.allclose(got, ref, atol=1e-5)
    got_c = Hn.attn_torch(q, k[:, :, :], v, True)
    ref_c = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert torch.allclose(got_c, ref_c, atol=1e-5)


def test_pivot_layout():
    recs = [({"mode": "fwd", "is_causal": True, "func_name": "a", "shape": [1, 1, 4, 8], "dtype": "bf16"}, ["1.50", "1", "2"]),
            ({"mode": "fwd", "is_causal": True, "func_name": "a", "shape": [1, 1, 16, 8], "dtype": "bf16"}, ["2.50", "1", "2"])]
    txt = Hn.pivot(recs, Hn._entry_bench)
    lines = txt.splitlines()
    assert "L=04,D=bf16" in lines[0] and "L=16,D=bf16" in lines[0]
    assert lines[1].startswith("Mode=fwd,C=True,F=a") and "1.50" in lines[1] and "2.50" in lines[1]


def test_varlen_ids_mark_sequences():
    """Packed-batch ids: one negative id per sequence, empty sequences skipped, tokens behind the
    last boundary in a sequence of their own; two tokens see each other iff their ids are equal,
    which is the block-diagonal mask of the packed batch (brute force)."""
    import torch
    from flash_mi355 import varlen_ids
    cu = torch.tensor([0, 3, 3, 7, 8], dtype=torch.int32)
    ids = varlen_ids(cu, 10)
    assert ids.dtype == torch.int32 and (ids < 0).all()
    want = [0, 0, 0, 2, 2, 2, 2, 3, 4, 4]          # sequence number of every token
    for i in range(10):
        for j in range(10):
            assert bool(ids[i] == ids[j]) == (want[i] == want[j])


def test_varlen_positions_align_sequences_bottom_right():
    """Packed causal positions: row i of sequence s sits at packed key i + (end of the sequence's keys
    - end of its queries), so the last query of every sequence sees exactly its last key; rows of a
    sequence with fewer keys than queries that see nothing land before the sequence's first key."""
    import torch
    from flash_mi355 import varlen_positions
    lq, lk = [4, 1, 0, 6, 3], [4, 9, 2, 8, 1]
    cq = torch.tensor([0] + list(torch.tensor(lq).cumsum(0)), dtype=torch.int32)
    ck = torch.tensor([0] + list(torch.tensor(lk).cumsum(0)), dtype=torch.int32)
    pos = varlen_positions(cq, ck, int(cq[-1]))
    assert pos.dtype == torch.int32 and pos.shape == (14,)
    for s in range(5):
        for t in range(lq[s]):
            i = int(cq[s]) + t
            want = int(ck[s]) + t + (lk[s] - lq[s])            # bottom-right: local row t sees local keys <= t + (lk - lq)
            assert int(pos[i]) == max(want, -1)
    assert int(pos[int(cq[4])]) < int(ck[4])                   # first rows of the last sequence (3 queries, 1 key): no key
    same = varlen_positions(cq, cq, int(cq[-1]))
    assert torch.equal(same, torch.arange(14, dtype=torch.int32))
