"""The host half of `Trainer::train_batch` / `train_chunk` in the C ABI (integer work, no device):
`ft_train_batch_select`, `ft_train_batch_plan`, `ft_chunk_padded_len`, `ft_pad_chunk` against literal
expected arrays typed from trainer/src/lib.rs:371-450 and against the oracle's restatement, bit for bit."""
import numpy as np
import pytest

from ferrotensor_amd import trainer as hip
from ferrotensor_amd._lib import FtError
from oracle import reference_step as rs


def test_select_cuts_at_the_attention_mask_and_drops_rows_that_cannot_train():
    ids = np.arange(40, dtype=np.uint32).reshape(5, 8)
    attn = np.array([[1, 1, 1, 1, 1, 0, 0, 0],     # 5 tokens, supervised inside: kept
                     [1, 0, 1, 1, 1, 1, 1, 1],     # cut at the first 0: one token left, dropped
                     [1, 1, 1, 1, 1, 1, 1, 1],     # full length, no supervised position: dropped
                     [1, 1, 1, 0, 0, 0, 0, 0],     # supervised only past the cut: dropped
                     [1, 1, 2, 1, 1, 1, 1, 1]],    # a flag other than 1 ends the row too: 2 tokens, kept
                    np.uint8)
    mask = np.array([[0, 0, 1, 1, 0, 1, 1, 1],
                     [1, 1, 1, 1, 1, 1, 1, 1],
                     [0, 0, 0, 0, 0, 0, 0, 0],
                     [0, 0, 0, 1, 1, 1, 1, 1],
                     [0, 7, 0, 0, 0, 0, 0, 0]], np.uint8)
    want = [5, 0, 0, 0, 2]
    assert rs.select_sequences(attn, mask) == want
    assert hip.select_sequences(ids, ids, attn, mask) == want


def test_select_matches_the_oracle_on_random_batches():
    rng = np.random.default_rng(0)
    for _ in range(50):
        B, S = int(rng.integers(1, 9)), int(rng.integers(1, 40))
        attn = (rng.random((B, S)) < 0.9).astype(np.uint8)
        mask = (rng.random((B, S)) < 0.2).astype(np.uint8)
        ids = rng.integers(0, 1000, (B, S)).astype(np.uint32)
        assert hip.select_sequences(ids, ids, attn, mask) == rs.select_sequences(attn, mask)


@pytest.mark.parametrize("n,accum,start,want", [
    (8, 4, 0, [4, 4]),
    (8, 4, 1, [3, 4, 1]),          # the open window takes 3 more, then a full one, then the rest
    (5, 8, 0, [5]),
    (5, 8, 6, [2, 3]),
    (3, 1, 0, [1, 1, 1]),
    (3, 2, 5, [1, 2]),             # a counter past the boundary: saturating_sub, then max(1)
    (0, 4, 0, []),
    (1, 4, 3, [1]),
])
def test_plan_stops_every_chunk_at_the_accumulation_boundary(n, accum, start, want):
    assert rs.plan_chunks(n, accum, start) == want
    assert hip.plan_chunks(n, accum, start) == want


def test_plan_without_an_accumulation_window_is_one_chunk():
    assert hip.plan_chunks(7, 0, 0) == [7]
    assert hip.plan_chunks(0, 0, 0) == []


def test_padding_pads_with_the_last_token_to_the_bucket():
    seqs = [([5, 6, 7], [6, 7, 8], [0, 1, 1]),
            ([1, 2, 3, 4, 5], [2, 3, 4, 5], [1, 1]),        # targets shorter: cut to 4; mask shorter: zeros
            ([9], [9, 9], [1])]
    rows, targets, masks = hip.pad_chunk(seqs, length_bucket=4)
    np.testing.assert_array_equal(rows, [[5, 6, 7, 7], [1, 2, 3, 4], [9, 9, 9, 9]])
    np.testing.assert_array_equal(targets, [[6, 7, 8, 7], [2, 3, 4, 5], [9, 9, 9, 9]])
    np.testing.assert_array_equal(masks, [[0, 1, 1, 0], [1, 1, 0, 0], [1, 0, 0, 0]])
    assert rows.dtype == np.uint32 and targets.dtype == np.uint32 and masks.dtype == np.uint8


def test_padding_matches_the_oracle_bit_for_bit():
    rng = np.random.default_rng(1)
    for bucket in (1, 8, 32):
        for _ in range(30):
            seqs = []
            for _ in range(int(rng.integers(1, 7))):
                n, m = int(rng.integers(1, 70)), int(rng.integers(1, 70))
                seqs.append((rng.integers(0, 49152, n).astype(np.uint32), rng.integers(0, 49152, m).astype(np.uint32),
                             rng.integers(0, 2, int(rng.integers(0, 70))).astype(np.uint8)))
            got = hip.pad_chunk(seqs, bucket)
            want = rs.pad_chunk([(list(i), list(t), list(m)) for i, t, m in seqs], bucket)
            for g, w in zip(got, want):
                assert g.dtype == w.dtype and g.shape == w.shape
                np.testing.assert_array_equal(g, w)


def test_a_row_longer_than_the_padded_length_is_refused():
    import ctypes as C
    from ferrotensor_amd import _lib
    lib = _lib.load()
    ids = np.arange(5, dtype=np.uint32)
    mk = np.ones(5, np.uint8)
    ptr = lambda a: (C.c_void_p * 1)(a.ctypes.data)
    n5 = (C.c_size_t * 1)(5)
    out32, out8 = np.zeros(4, np.uint32), np.zeros(4, np.uint8)
    rc = lib.ft_pad_chunk(ptr(ids), ptr(ids), ptr(mk), n5, n5, n5, 1, 4, out32.ctypes.data_as(C.c_void_p),
                          out32.ctypes.data_as(C.c_void_p), out8.ctypes.data_as(C.c_void_p))
    assert rc != 0 and b"5 tokens" in lib.ft_last_error()
    with pytest.raises(FtError):
        _lib.check(rc)
