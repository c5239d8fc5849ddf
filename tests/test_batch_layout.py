"""The packed step metadata: rows, sequences and wanted rows of a mixed batch, as the library's
batch builder lays them out (driven without a GPU through its host-object calls)."""
from types import SimpleNamespace

import pytest

from celeg_amd.engine import StepEntry
from celeg_amd.native import HostError, HostObject


def build(entries, pad_to=None, updates=((),), caps=None):
    builder = HostObject("batch", capacity=4096, n_groups=len(updates))
    options = {"null_slot": 9}
    if pad_to is not None:
        options["pad_to"] = pad_to
    if caps is not None:
        options["update_caps"] = list(caps)
    out = builder.call("build", [{"slot": e.slot, "start_pos": e.start_pos, "tokens": list(e.tokens),
                                  "want": list(e.want)} for e in entries],
                       [[list(u) for u in g] for g in updates], options)
    return SimpleNamespace(**out)


def test_single_tokens_lie_first_and_logits_keep_the_entries_order():
    entries = [StepEntry(3, 10, [5, 6, 7], [2]), StepEntry(1, 40, [8], [0]),
               StepEntry(2, 0, [1, 2], [0, 1]), StepEntry(0, 7, [9], [0])]
    b = build(entries)
    assert (b.n_tokens, b.n_seqs, b.single_rows, b.decode_only) == (7, 4, 2, False)
    assert b.entry_order == [1, 3, 0, 2]
    assert b.token_ids == [8, 9, 5, 6, 7, 1, 2]
    assert b.positions == [40, 7, 10, 11, 12, 0, 1]
    assert b.token_slot == [1, 0, 3, 3, 3, 2, 2]
    assert b.token_seq == [0, 1, 2, 2, 2, 3, 3]
    assert b.cu_seqlens == [0, 1, 2, 5, 7]
    assert b.seq_slot == [1, 0, 3, 2] and b.seq_start == [40, 7, 10, 0]
    # wanted rows in the order of the entries and of their ``want``
    assert b.logit_rows == [4, 0, 5, 6, 1]


def test_single_rows_only_and_padding():
    entries = [StepEntry(2, 5, [11], [0]), StepEntry(0, 9, [12], [0])]
    b = build(entries)
    assert b.decode_only and b.single_rows == 2 and b.entry_order == [0, 1]
    b = build(entries, pad_to=4)
    assert (b.n_tokens, b.n_seqs, b.single_rows) == (4, 4, 4)
    assert b.token_slot == [2, 0, 9, 9] and b.logit_rows == [0, 1, 2, 3]


def test_a_portion_alone_has_no_single_rows():
    b = build([StepEntry(0, 0, [1, 2, 3, 4], [3])])
    assert b.single_rows == 0 and b.logit_rows == [3]


def test_attention_rows_kernel_fits_lds_at_the_longest_context():
    """What the prefill attention asks of LDS at a block table of 8,000 entries (a context of
    128,000 tokens in pages of 16) for every head size and form: within the 160 KB of a
    compute unit, because a tile keeps at most 4,096 entries of its request's table there."""
    import ctypes
    from celeg_amd.csrc import build as library
    lib = ctypes.CDLL(library.ensure_built())
    lib.celeg_attention_rows_lds_bytes.restype = ctypes.c_longlong
    for head_dim in (32, 64, 96, 128):
        for sets in (1, 2) + ((4,) if head_dim <= 64 else ()):      # (four sets: heads up to 64)
            for stride in (8, 256, 4096, 8000, 1 << 20):
                need = lib.celeg_attention_rows_lds_bytes(head_dim, sets, stride)
                assert 0 < need <= 160 * 1024, (head_dim, sets, stride, need)


def test_table_updates_travel_in_the_same_buffer_and_arrays_start_at_multiples_of_four():
    entries = [StepEntry(1, 0, [4, 5, 6], [2])]
    b = build(entries, updates=([(1, 0, 7)], [(1, 0, 3), (1, 1, 4)]), caps=(4, 2))
    assert b.table_updates[0] == [1, 1, 0, 7] + [0] * 9 or b.table_updates[0][:4] == [1, 1, 0, 7]
    assert b.table_updates[1][:7] == [2, 1, 0, 3, 1, 1, 4]
    assert all(off % 4 == 0 for off in b.offsets)
    with pytest.raises(HostError, match="more block-table updates"):
        build(entries, updates=([(1, 0, 7), (1, 1, 8)],), caps=(1,))
    with pytest.raises(HostError, match="wanted place"):
        build([StepEntry(1, 0, [4, 5, 6], [3])])
    with pytest.raises(HostError, match="padded"):
        build(entries, pad_to=4)


def test_the_products_for_up_to_64_rows_share_out_their_columns():
    """The products for 9 to 64 rows and for up to 16 say how many columns a workgroup owns and how
    many workgroups that makes: together the shares cover every column once; a share never exceeds
    the 64 columns a workgroup's tiles can hold; and where a share is smaller than a tile of 16
    columns (few columns: the share is halved so that more compute units get a workgroup), the
    workgroups of all row groups still fit the chip's 256 compute units at once."""
    import ctypes
    from celeg_amd.csrc import build as library
    lib = ctypes.CDLL(library.ensure_built())
    epilogues = {"store": 0, "store_f32": 1, "residual": 2, "swiglu": 3, "conv": 4}
    for name, epi in epilogues.items():
        for n in (24, 333, 1024, 2048, 3072, 4608, 7168, 65536):
            for k in (64, 1024, 4608):
                for m in range(1, 65):
                    cols, blocks = lib.celeg_gemm_rows_cols(m, n, k, epi), lib.celeg_gemm_rows_blocks(m, n, k, epi)
                    assert 1 <= cols <= 64 and (blocks - 1) * cols < n <= blocks * cols, (name, m, n, k, cols, blocks)
                    groups = lib.celeg_gemm_rows_workgroups(m, n, k, epi)
                    assert groups % blocks == 0 and 1 <= groups // blocks <= (m + 15) // 16
                    if cols < 16:
                        assert groups <= 256, (name, m, n, k, cols, blocks, groups)
                if name != "conv" or k % 8 == 0:
                    for m in range(1, 17):
                        cols, blocks = lib.celeg_gemv_slices_cols(m, n, k), lib.celeg_gemv_slices_blocks(m, n, k)
                        assert cols >= 1 and (blocks - 1) * cols < n <= blocks * cols, (m, n, k, cols, blocks)
