"""Host-side helpers of the launchers (no GPU): what a launcher remembers about a set of tables, and the
padded receive buffer of the chunked reduce."""

import gc

import torch

from syncopate_amd.computation._launch import already_checked, recall_note, remember_checked, remember_note
from syncopate_amd.computation.reduce import RECEIVE_BLOCK_PAD_BYTES, padded_receive_buffer


def _tables():
    return tuple(torch.arange(4 * (i + 1), dtype=torch.int32) for i in range(4))


def test_notes_are_kept_per_objects_and_versions():
    tables = _tables()
    assert recall_note(tables, "form") is None
    remember_note(tables, "form", (True, 12))
    remember_note(tables, "programs", 12)
    assert recall_note(tables, "form") == (True, 12) and recall_note(tables, "programs") == 12
    # other objects with the same contents: nothing is known about them
    assert recall_note(_tables(), "form") is None
    # an in-place write to any of the tables voids every note about the set
    tables[2][0] = 7
    assert recall_note(tables, "form") is None and recall_note(tables, "programs") is None
    remember_note(tables, "form", (False, 0))
    assert recall_note(tables, "form") == (False, 0)


def test_a_note_does_not_outlive_its_tables():
    """Ids are reused once an object is gone: a note is tied to the objects (weak references), not to their ids."""
    tables = _tables()
    remember_note(tables, "form", "old")
    ids = tuple(id(t) for t in tables)
    del tables
    gc.collect()
    for _ in range(64):                       # give the allocator a chance to hand the ids out again
        fresh = _tables()
        if tuple(id(t) for t in fresh) == ids:
            assert recall_note(fresh, "form") is None
            break
        assert recall_note(fresh, "form") is None


def test_checked_tables_cache_matches_parameters():
    tables = _tables()
    assert not already_checked(tables, (1, 2))
    remember_checked(tables, (1, 2))
    assert already_checked(tables, (1, 2)) and not already_checked(tables, (1, 3))
    tables[0].add_(1)
    assert not already_checked(tables, (1, 2))


def test_padded_receive_buffer_layout():
    world, rows, n = 8, 16, 64
    buf = padded_receive_buffer(world, rows, n, torch.bfloat16, "cpu")
    pad = RECEIVE_BLOCK_PAD_BYTES // 2
    assert buf.shape == (world, rows, n) and buf.stride() == (rows * n + pad, n, 1)
    assert buf[3].is_contiguous() and not buf.is_contiguous()
    # blocks do not overlap: a write to one leaves the others alone
    buf.zero_()
    buf[3].fill_(1.0)
    assert buf.sum().item() == rows * n
    assert buf[4].data_ptr() - buf[3].data_ptr() == (rows * n + pad) * 2
    one = padded_receive_buffer(1, rows, n, torch.float16, "cpu")
    assert one.shape == (1, rows, n)


def test_tile_policy_picks_a_shape_whose_last_chunk_fills_the_machine():
    """The producer-bound regime of the all-gather GEMM: what is left to compute when the last chunk lands is
    `rounds x tile time` of that chunk's tiles (reference: the tile shape is a call-site kwarg,
    syncopate/computation/gemm/template.py:193-220, swept by hand in tests/test_ag_gemm_tile_size_sensitivity.py)."""
    import pytest

    from syncopate_amd.computation.gemm.tile_policy import choose_tile, rounds

    # headline shape: chunks of 1024 rows x 3584 columns on 224 programs
    assert rounds(1024, 3584, 256, 256, 224) == 1 and rounds(1024, 3584, 128, 128, 224) == 1
    assert choose_tile(1024, 3584, 224, producer_bound=False) == (256, 256)
    assert choose_tile(1024, 3584, 224, producer_bound=True) == (256, 128)
    # a chunk that is many rounds of any shape: the cheapest per element wins either way
    assert choose_tile(8192, 8192, 224, producer_bound=True) == (256, 256)
    # only shapes that divide the chunk are offered
    assert choose_tile(128, 256, 224, producer_bound=True) in ((128, 256), (128, 128))
    assert choose_tile(1024, 3584, 224, producer_bound=True, shapes=[(256, 256), (128, 128)]) == (128, 128)
    with pytest.raises(ValueError):
        choose_tile(100, 3584, 224, producer_bound=True)


def test_trusted_flag_arrays_are_remembered_per_tensor_object():
    """Launchers fence behind every flag wait unless the flag array has been declared trusted
    (include/syncopate_hip.h, SYN_GEMM_ACQUIRE_ALWAYS); the declaration is for the tensor object, not for its
    address or for views of it, and goes away with the tensor."""
    import gc

    import torch

    from syncopate_amd.computation._launch import acquire_always, trust_flags

    flags = torch.zeros(8, dtype=torch.int64)
    other = torch.zeros(8, dtype=torch.int64)
    assert acquire_always(flags) and acquire_always(other)
    trust_flags(flags)
    assert not acquire_always(flags)
    assert acquire_always(other)
    assert acquire_always(flags[2:])            # a view is another object: the conservative answer
    key = id(flags)
    del flags
    gc.collect()
    later = torch.zeros(8, dtype=torch.int64)
    assert acquire_always(later)                 # whatever object now lives at that id is not trusted
    from syncopate_amd.computation import _launch
    assert key not in _launch._trusted_flags or _launch._trusted_flags.get(key) is None


def test_xcd_remap_policy_follows_the_measurements():
    """Smaller tiles gain from the remap, the 256 x 256 tile does not (and loses with 256 programs): a launcher that was
    not told takes it for the former only."""
    from syncopate_amd.computation.gemm.tile_policy import choose_xcd_remap

    assert not choose_xcd_remap(256, 256)
    assert all(choose_xcd_remap(bm, bn) for bm, bn in ((128, 256), (256, 128), (128, 128), (256, 224)))
