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


class _Tok:
    vocab_size, eos_token_id = 1000, 2

    def __len__(self):
        return 1001  # the collator pads with len(tokenizer) - 1


def _write_json(path, docs):
    import json
    with open(path, "w") as f:
        for d in docs:
            f.write(json.dumps({"input_ids": d}) + "\n")


def test_cache_built_from_json_lines_equals_the_cache_built_from_token_arrays(tmp_path):
    rng = np.random.RandomState(7)
    docs = [rng.randint(3, 1000, size=int(rng.randint(1, 50))).tolist() + [2] for _ in range(23)]
    docs.insert(5, [])  # an empty document is skipped (data_utils.py:372-373)
    _write_json(tmp_path / "a.jsonl", docs[:10])
    _write_json(tmp_path / "b.jsonl", docs[10:])
    direct = _write_cache(tmp_path, [d for d in docs if d])
    for workers, splits, name in ((1, 1, "one"), (2, 1, "pool"), (1, 2, "split_files")):
        prefix = str(tmp_path / name)
        n = M.build_data_cache(M.encode_tokenised_line, 1000, [str(tmp_path / "a.jsonl"), str(tmp_path / "b.jsonl")], prefix,
                               cache_worker=workers, cache_splits=splits)
        assert n == 23
        for ext in (".idx", ".bin"):
            assert open(prefix + ext, "rb").read() == open(direct + ext, "rb").read(), (name, ext)
    # a single file split by lines into three parts, built part by part, merged
    _write_json(tmp_path / "all.jsonl", docs)
    prefix = str(tmp_path / "split_lines")
    M.build_data_cache(M.encode_tokenised_line, 1000, str(tmp_path / "all.jsonl"), prefix, cache_worker=1, cache_splits=3)
    for ext in (".idx", ".bin"):
        assert open(prefix + ext, "rb").read() == open(direct + ext, "rb").read()
    assert M.split_list(list(range(7)), 3) == [[0, 1, 2], [3, 4], [5, 6]]
    with pytest.raises(RuntimeError):  # a stray .bin without its .idx is never overwritten
        open(str(tmp_path / "stray.bin"), "wb").close()
        M.build_data_cache(M.encode_tokenised_line, 1000, str(tmp_path / "a.jsonl"), str(tmp_path / "stray"), cache_worker=1)


def test_json_dataset_builds_its_cache_once_and_feeds_the_collator(tmp_path):
    from easyllm_amd import data as D
    rng = np.random.RandomState(11)
    docs = [rng.randint(3, 1000, size=int(rng.randint(2, 40))).tolist() + [2] for _ in range(60)]
    _write_json(tmp_path / "train.jsonl", docs)
    seq = 64
    kw = dict(data_root=str(tmp_path), seed=5, total_samples=8, max_seq_length=seq, tokenizer=_Tok(), cache_worker=1,
              with_cu_lens=True)
    ds = M.MMapIndexJsonDataset(json_file=str(tmp_path / "train.jsonl"), **kw)
    assert os.path.exists(str(tmp_path / "train_data_cache" / "mmap_sentebnse.idx"))
    again = M.MMapIndexJsonDataset(**kw)  # the cache exists: no json needed
    assert torch.equal(ds[3]["input_ids"], again[3]["input_ids"])
    with pytest.raises(AssertionError):
        M.MMapIndexJsonDataset(str(tmp_path / "elsewhere"), 5, 8, seq, tokenizer=_Tok())
    # a transformer that maps parsed json to tokens is applied per line
    doubled = M.MMapIndexJsonDataset(json_file=str(tmp_path / "train.jsonl"), cache_prefix="doubled",
                                     transformer=lambda meta: {"input_ids": torch.tensor(meta["input_ids"] * 2)}, **kw)
    assert doubled._index.sizes.tolist() == [2 * len(d) for d in docs]
    # collator: next-token shift, boundaries clamped to the sequence length and flattened over the batch
    items = [ds[0], ds[1]]
    batch = D.batch_align_collate(items, pad_token_id=1000, max_seq_length=seq, pretrain=True)
    for b, it in enumerate(items):
        assert batch["input_ids"][b].tolist() == it["input_ids"][:-1].tolist()
        assert batch["labels"][b].tolist() == it["input_ids"][1:].tolist()
        assert batch["position_ids"][b].tolist() == it["position_ids"][:-1].tolist()
    want = O.flatten_cu_seqlens([it["cu_seqlens"].tolist() for it in items], seq)
    assert batch["cu_seqlens"].tolist() == want.tolist() and batch["cu_seqlens"][-1].item() == 2 * seq
    (tokens, pos, mask, cu), (labels, loss_mask) = D.flash_batch_from(batch, pad_token_id=1000, pretrain=True)
    assert mask.all() and loss_mask.dtype == torch.bool and torch.equal(cu, batch["cu_seqlens"])
    # ragged items without the packed fields: padded with the pad token / ignore index to the longest, shifted
    short = {"input_ids": torch.tensor([5, 6, 7]), "labels": torch.tensor([5, 6, 7])}
    long_ = {"input_ids": torch.tensor([8, 9, 10, 11, 12]), "labels": torch.tensor([8, 9, 10, 11, 12])}
    b2 = D.batch_align_collate([short, long_], pad_token_id=1000, max_seq_length=seq, alignment=4)
    assert b2["input_ids"].tolist() == [[5, 6, 1000, 1000, 1000, 1000, 1000, 1000], [8, 9, 10, 11, 1000, 1000, 1000, 1000]]
    assert b2["labels"].tolist() == [[6, 7, -100, -100, -100, -100, -100, -100], [9, 10, 11, 12, -100, -100, -100, -100]]
