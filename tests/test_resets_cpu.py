"""Host logic of the length / new_starts wrapper: the packed-sequence table it builds
(/root/reference/rwkv_ops/rwkv7_kernel/cuda_kernel/wkv7_jax.cu:18,23-24,46-51,66 for what the two arguments mean)."""
import pytest

from rwkv_ops_amd.rwkv7.resets import cu_seqlens_from_resets


def test_plain_batch_is_one_sequence_per_row():
    cu, first, last = cu_seqlens_from_resets(3, 10)
    assert cu == [0, 10, 20, 30] and first == [0, 1, 2] and last == [0, 1, 2]


def test_lengths_cut_the_padding_off():
    cu, first, last = cu_seqlens_from_resets(3, 10, length=[10, 4, 0])
    # row 1: tokens 10..13 valid, 14..19 a sequence of their own; row 2: nothing valid
    assert cu == [0, 10, 14, 20, 30]
    assert first == [0, 1, 3] and last == [0, 1, -1]


def test_new_starts_split_rows_and_drop_the_initial_state():
    ns = [[False] * 8 for _ in range(2)]
    ns[0][3] = True
    ns[1][0] = True
    ns[1][5] = True
    cu, first, last = cu_seqlens_from_resets(2, 8, length=[8, 5], new_starts=ns)
    assert cu == [0, 3, 8, 13, 16]
    assert first == [0, -1]             # row 1 restarts at its first token: its initial state is not used
    assert last == [1, 2]               # row 0 ends with its second document, row 1 after token 4 (a cut and a reset there)


def test_bad_arguments():
    with pytest.raises(ValueError):
        cu_seqlens_from_resets(2, 8, length=[8])
    with pytest.raises(ValueError):
        cu_seqlens_from_resets(2, 8, length=[8, 9])
    with pytest.raises(ValueError):
        cu_seqlens_from_resets(2, 8, new_starts=[[False] * 8])
