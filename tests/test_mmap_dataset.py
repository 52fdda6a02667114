"""Packed-sequence token cache: native sample-location builder against the oracle's closed form and the reference's own
compiled helper (when oracle/_ref has been built), index file format, and sample extraction."""
import os
import struct

import numpy as np
import pytest
import torch

from oracle import build_ref, llama_oracle as O
from easyllm_amd import mmap_dataset as M


def _case(seed, ndocs, lo, hi, seq, epochs):
    rng = np.random.RandomState(seed)
    sizes = rng.randint(lo, hi + 1, size=ndocs).astype(np.int32)
    if sizes.sum() < 2:
        sizes[0] += 2
    doc_idx = np.concatenate([rng.permutation(ndocs) for _ in range(epochs)]).astype(np.int32)
    return sizes, doc_idx, seq, epochs, int(sizes.sum())


CASES = [_case(1, 50, 1, 40, 16, 1), _case(2, 7, 0, 9, 5, 3), _case(3, 200, 1, 700, 128, 2), _case(4, 3, 1, 3, 2, 4),
         _case(5, 1, 1000, 1000, 64, 1), _case(6, 30, 8, 8, 8, 2)]  # last: every boundary falls on a document's last token


@pytest.mark.parametrize("case", CASES)
def test_native_location_idx_matches_closed_form_and_reference_helper(case):
    sizes, doc_idx, seq, epochs, tpe = case
    got = M.build_location_idx(sizes, doc_idx, seq, epochs, tpe)
    want = O.build_location_idx(sizes, doc_idx, seq, epochs, tpe)
    assert got.dtype == np.int32 and got.shape == ((epochs * tpe - 1) // seq + 1, 2)
    assert np.array_equal(got, want)
    ref = build_ref.load()
    if ref is not None:  # the reference's helpers.cpp, compiled in place
        assert np.array_equal(np.asarray(ref.build_location_idx(sizes, doc_idx, seq, epochs, tpe)), got)
    # brute force: the tokens of sample k are stream[k*seq : k*seq + seq + 1]
    stream_doc = np.concatenate([np.full(sizes[d], i) for i, d in enumerate(doc_idx)])
    stream_off = np.concatenate([np.arange(sizes[d]) for d in doc_idx])
    for k in range(got.shape[0]):
        assert (stream_doc[k * seq], stream_off[k * seq]) == tuple(got[k])


@pytest.fixture(scope="module", autouse=True)
def _reference_helper():
    """Where the reference tree is present, make sure its helper has been compiled into oracle/_ref (normally done by
    __graft_entry__.build()); elsewhere the prebuilt module is used if it travelled with the tree."""
    if build_ref.load() is None and os.path.exists(build_ref.REF_SRC):
        build_ref.build(verbose=False)
    yield


def test_reference_helper_is_available_where_the_reference_tree_is():
    if os.path.exists(build_ref.REF_SRC):
        assert build_ref.load() is not None


def test_native_location_idx_rejects_bad_input():
    sizes = np.array([4, 4], dtype=np.int32)
    with pytest.raises(ValueError):
        M.build_location_idx(sizes, np.array([0, 1], dtype=np.int32), 1, 1, 8)       # seq_length must exceed 1
    with pytest.raises(RuntimeError):
        M.build_location_idx(sizes, np.array([0, 5], dtype=np.int32), 4, 1, 8)       # document id out of range
    with pytest.raises(RuntimeError):
        M.build_location_idx(sizes, np.array([0, 1], dtype=np.int32), 4, 2, 8)       # claims 16 tokens, holds 8


def _write_cache(tmp_path, docs, dtype=np.uint16):
    prefix = str(tmp_path / "cache")
    b = M.MMapIndexedDatasetBuilder(M.data_file_path(prefix), dtype=dtype)
    for d in docs:
        b.add_item(torch.tensor(d))
        b.end_document()
    b.finalize(M.index_file_path(prefix))
    return prefix


def test_index_file_format_round_trip(tmp_path):
    docs = [[5, 6, 7], [8], [9, 10, 11, 12]]
    prefix = _write_cache(tmp_path, docs, dtype=np.uint16)
    raw = open(M.index_file_path(prefix), "rb").read()
    assert raw[:9] == b"MMIDIDX\x00\x00" and struct.unpack("<Q", raw[9:17]) == (1,) and raw[17] == 8  # uint16 has code 8
    assert struct.unpack("<QQ", raw[18:34]) == (3, 4)
    idx = M.MMapIndex(M.index_file_path(prefix))
    assert idx.dtype == np.uint16 and idx.sizes.tolist() == [3, 1, 4] and idx.doc_idx.tolist() == [0, 1, 2, 3]
    assert [int(idx[i][0]) for i in range(3)] == [0, 6, 8]  # byte pointers
    assert np.fromfile(M.data_file_path(prefix), dtype=np.uint16).tolist() == [5, 6, 7, 8, 9, 10, 11, 12]
    assert M.best_fitting_dtype(32000) == np.uint16 and M.best_fitting_dtype(152064) == np.int32


def test_dataset_samples_are_windows_of_the_document_stream(tmp_path):
    rng = np.random.RandomState(0)
    eos = 2
    docs = []
    for _ in range(40):
        n = int(rng.randint(3, 60))
        docs.append(rng.randint(3, 1000, size=n - 1).tolist() + [eos])
    prefix = _write_cache(tmp_path, docs)
    seq, total = 32, 70  # more than one epoch
    ds = M.MMapIndexDataset(prefix, seed=123, total_samples=total, max_seq_length=seq, eos_token_id=eos, with_cu_lens=True,
                            shuffle=False)
    stream = np.concatenate([np.asarray(docs[d]) for d in ds.sentenses_idx])
    assert len(ds) >= total
    for k in (0, 1, len(ds) // 2, len(ds) - 1):
        item = ds[k]
        assert item["input_ids"].tolist() == stream[k * seq:k * seq + seq + 1].tolist() and torch.equal(item["labels"], item["input_ids"])
        cu = item["cu_seqlens"].tolist()
        assert cu == O.get_cu_seqlens(item["input_ids"], eos) and cu[0] == 0 and cu[-1] == seq + 1
        assert item["position_ids"].tolist() == O.get_position_ids(cu)
    # epochs are shuffled together (the last one apart when it is short): every document appears once per epoch overall;
    # the shuffled view visits every sample exactly once
    counts = np.bincount(np.asarray(ds.sentenses_idx), minlength=len(docs))
    assert counts.min() == counts.max() == len(ds.sentenses_idx) // len(docs) >= 2
    shuffled = M.MMapIndexDataset(prefix, seed=123, total_samples=total, max_seq_length=seq)
    assert sorted(np.asarray(shuffled.shuffle_idx).tolist()) == list(range(len(shuffled)))
    again = M.MMapIndexDataset(prefix, seed=123, total_samples=total, max_seq_length=seq)
    assert np.array_equal(again.shuffle_idx, shuffled.shuffle_idx) and np.array_equal(again.sentenses_idx, shuffled.sentenses_idx)
    assert M.num_epochs_for(100, 10, 9) == 1 and M.num_epochs_for(100, 10, 10) == 2  # (100 - 1) // 10 = 9 samples per epoch
    with pytest.raises(FileNotFoundError):
        M.MMapIndexDataset(str(tmp_path / "missing"), 1, 1, 8)
