"""Packed-sequence dataset over the reference's on-disk token cache (`<prefix>.idx` + `<prefix>.bin`).

Counterpart of llm/data/data_utils.py:106-260 (`MMapIndex`, `MMapIndexedDatasetBuilder`: header magic `MMIDIDX\\0\\0`,
version 1, dtype code, sizes int32, byte pointers int64, document index int64) and of `MMapIndexJsonDataset`
(llm/data/nlp_dataset.py:322-646) from the point where the token cache exists: the three index maps (document order
per epoch, sample locations, sample shuffle), sample extraction, and `cu_seqlens` / `position_ids` emission for the
packed attention path.  `build_data_cache` writes the cache from line-json files (data_utils.py:268-385): every line
goes through an `encode` callable -- the reference's tokenizer + transform pipeline, which is not part of this build, or
by default a reader of already tokenised lines `{"input_ids": [...]}` -- and becomes one document of the cache.

The sample-location table comes from the native builder (`ezl_build_location_idx`), which replaces the reference's
pybind11 helper; there is no python fallback for it.
"""
import json
import os
import shutil
import struct
import tempfile
from multiprocessing import Pool

import numpy as np
import torch

from . import _lib
from .data import get_cu_seqlens, get_position_ids

DTYPES = {1: np.uint8, 2: np.int8, 3: np.int16, 4: np.int32, 5: np.int64, 6: np.float32, 7: np.double, 8: np.uint16}
_HDR_MAGIC = b"MMIDIDX\x00\x00"


def index_file_path(prefix_path):
    return prefix_path + ".idx"


def data_file_path(prefix_path):
    return prefix_path + ".bin"


def best_fitting_dtype(vocab_size=None):
    return np.uint16 if vocab_size is not None and vocab_size < 65500 else np.int32


def dtype_code(dtype):
    for k, v in DTYPES.items():
        if v == dtype:
            return k
    raise ValueError(dtype)


class MMapIndex:
    """Reader of `<prefix>.idx`; `MMapIndex.write(path, dtype, sizes, doc_idx)` writes one."""

    @staticmethod
    def write(path, dtype, sizes, doc_idx):
        sizes32 = np.asarray(sizes, dtype=np.int32)
        pointers = np.zeros(len(sizes32), dtype=np.int64)
        if len(sizes32) > 1:
            np.cumsum(sizes32[:-1].astype(np.int64) * np.dtype(dtype).itemsize, out=pointers[1:])
        with open(path, "wb") as f:
            f.write(_HDR_MAGIC)
            f.write(struct.pack("<Q", 1))
            f.write(struct.pack("<B", dtype_code(dtype)))
            f.write(struct.pack("<Q", len(sizes32)))
            f.write(struct.pack("<Q", len(doc_idx)))
            f.write(sizes32.tobytes(order="C"))
            f.write(pointers.tobytes(order="C"))
            f.write(np.asarray(doc_idx, dtype=np.int64).tobytes(order="C"))

    def __init__(self, path, skip_warmup=True):
        with open(path, "rb") as stream:
            assert stream.read(9) == _HDR_MAGIC, "Index file doesn't match expected format."
            assert struct.unpack("<Q", stream.read(8)) == (1,)
            (code,) = struct.unpack("<B", stream.read(1))
            self._dtype = DTYPES[code]
            self._len = struct.unpack("<Q", stream.read(8))[0]
            self._doc_count = struct.unpack("<Q", stream.read(8))[0]
            offset = stream.tell()
        self._mmap = np.memmap(path, mode="r", order="C")
        self._sizes = np.frombuffer(self._mmap, dtype=np.int32, count=self._len, offset=offset)
        self._pointers = np.frombuffer(self._mmap, dtype=np.int64, count=self._len, offset=offset + self._sizes.nbytes)
        self._doc_idx = np.frombuffer(self._mmap, dtype=np.int64, count=self._doc_count,
                                      offset=offset + self._sizes.nbytes + self._pointers.nbytes)

    dtype = property(lambda self: self._dtype)
    sizes = property(lambda self: self._sizes)
    doc_idx = property(lambda self: self._doc_idx)

    def __getitem__(self, i):
        return self._pointers[i], self._sizes[i]

    def __len__(self):
        return self._len


class MMapIndexedDatasetBuilder:
    """add_item(tokens) ... end_document() ... finalize(index_file): data_utils.py:218-255."""

    def __init__(self, out_file, dtype=np.int64):
        self._data_file = open(out_file, "wb")
        self._dtype = dtype
        self._sizes = []
        self._doc_idx = [0]

    def add_item(self, tensor):
        arr = np.array(tensor.numpy() if isinstance(tensor, torch.Tensor) else tensor, dtype=self._dtype)
        self._data_file.write(arr.tobytes(order="C"))
        self._sizes.append(arr.size)

    def end_document(self):
        self._doc_idx.append(len(self._sizes))

    def merge_file_(self, another_prefix):
        """Appends the cache `<another_prefix>.idx/.bin` (data_utils.py:234-248)."""
        index = MMapIndex(index_file_path(another_prefix))
        assert index.dtype == self._dtype
        offset = len(self._sizes)
        self._sizes.extend(int(x) for x in index.sizes)
        self._doc_idx.extend(int(x) for x in (offset + index.doc_idx)[1:])
        with open(data_file_path(another_prefix), "rb") as f:
            shutil.copyfileobj(f, self._data_file)

    def finalize(self, index_file):
        self._data_file.close()
        MMapIndex.write(index_file, self._dtype, self._sizes, self._doc_idx)


def split_list(lst, n):
    """n nearly equal consecutive parts (data_utils.py:258-264)."""
    k, m = divmod(len(lst), n)
    return [lst[i * k + min(i, m):(i + 1) * k + min(i + 1, m)] for i in range(n)]


def encode_tokenised_line(json_line):
    """Default `encode`: a line that already holds its token ids."""
    meta = json.loads(json_line)
    return {"input_ids": torch.as_tensor(meta["input_ids"], dtype=torch.int64)}


def _build_one_cache(encode, vocab_size, json_files, cache_prefix, cache_worker):
    """data_utils.py:333-385: one document per non-empty encoded line, in file and line order."""
    if os.path.exists(data_file_path(cache_prefix)) and os.path.exists(index_file_path(cache_prefix)):
        return 0
    if os.path.exists(data_file_path(cache_prefix)):
        raise RuntimeError("%s.bin already exists. Please manually remove it first" % cache_prefix)
    builder = MMapIndexedDatasetBuilder(data_file_path(cache_prefix), dtype=best_fitting_dtype(vocab_size))
    items = 0
    for jsf in json_files:
        with open(jsf, "r", encoding="utf-8") as fin:
            if cache_worker and cache_worker > 1:
                with Pool(cache_worker) as pool:
                    encoded = list(pool.imap(encode, fin, 25))
            else:
                encoded = [encode(line) for line in fin]
        for meta in encoded:
            ids = torch.as_tensor(meta["input_ids"]).int().cpu().numpy()
            if ids.size == 0:
                continue
            builder.add_item(ids)
            builder.end_document()
            items += 1
    builder.finalize(index_file_path(cache_prefix))
    return items


def build_data_cache(encode, vocab_size, json_file, cache_prefix, cache_worker=4, cache_splits=1, cache_indices=None):
    """Token cache `<cache_prefix>.idx/.bin` from line-json files (data_utils.py:268-330).  With cache_splits > 1 the files
    (or, for a single file, its lines) are cut into that many parts, each built as `<cache_prefix>_<i>` -- only the parts
    named in cache_indices, when given -- and, when all were built, merged in order into one cache."""
    assert cache_splits >= 1
    json_file = list(json_file) if isinstance(json_file, (list, tuple)) else [json_file]
    if cache_splits == 1:
        return _build_one_cache(encode, vocab_size, json_file, cache_prefix, cache_worker)
    temp_files = []
    if len(json_file) == 1:
        with open(json_file[0], "r", encoding="utf-8") as f:
            lines = f.readlines()
        assert len(lines) >= cache_splits
        json_file = []
        for part in split_list(lines, cache_splits):
            with tempfile.NamedTemporaryFile(mode="w+", delete=False) as tf:
                tf.writelines(part)
                json_file.append(tf.name)
                temp_files.append(tf.name)
    cache_splits = min(len(json_file), cache_splits)
    parts = split_list(json_file, cache_splits)
    items = 0
    try:
        for i, part in enumerate(parts):
            if cache_indices is not None and i not in cache_indices:
                continue
            items += _build_one_cache(encode, vocab_size, part, cache_prefix + "_%d" % i, cache_worker)
    finally:
        for name in temp_files:
            os.remove(name)
    if cache_indices is None:
        merged = MMapIndexedDatasetBuilder(data_file_path(cache_prefix), dtype=best_fitting_dtype(vocab_size))
        for i in range(len(parts)):
            merged.merge_file_(cache_prefix + "_%d" % i)
        merged.finalize(index_file_path(cache_prefix))
    return items


def num_epochs_for(tokens_per_epoch, seq_length, num_samples):
    """Epochs needed for num_samples samples of seq_length + 1 overlapping tokens (data_utils.py:88-103)."""
    num_epochs, total_tokens = 0, 0
    while True:
        num_epochs += 1
        total_tokens += tokens_per_epoch
        if (total_tokens - 1) // seq_length >= num_samples:
            return num_epochs


def build_location_idx(sizes, doc_idx, seq_length, num_epochs, tokens_per_epoch):
    """int32 [num_samples + 1, 2] through the native builder."""
    sizes = np.ascontiguousarray(sizes, dtype=np.int32)
    doc_idx = np.ascontiguousarray(doc_idx, dtype=np.int32)
    rows = _lib.location_idx_rows(int(seq_length), int(num_epochs), int(tokens_per_epoch))
    if rows <= 0:
        raise ValueError("need seq_length > 1, num_epochs > 0 and tokens_per_epoch > 1")
    out = np.zeros((rows, 2), dtype=np.int32)
    _lib.call("ezl_build_location_idx", sizes.ctypes.data, sizes.size, doc_idx.ctypes.data, doc_idx.size, int(seq_length),
              int(num_epochs), int(tokens_per_epoch), out.ctypes.data, rows)
    return out


def build_sentense_idx(sentense_id, num_epochs, np_rng, separate_last_epoch):
    """Document order over all epochs, shuffled; the last epoch separately when asked (nlp_dataset.py:409-422)."""
    if not separate_last_epoch or num_epochs == 1:
        idx = np.tile(np.asarray(sentense_id, dtype=np.int32), num_epochs)
        np_rng.shuffle(idx)
        return idx
    first = build_sentense_idx(sentense_id, num_epochs - 1, np_rng, False)
    last = build_sentense_idx(sentense_id, 1, np_rng, False)
    return np.concatenate((first, last))


def build_shuffle_idx(num_samples, total_size, np_rng):
    """[0, num_samples) shuffled, then [num_samples, total_size) shuffled (nlp_dataset.py:465-479)."""
    dtype_ = np.int64 if total_size >= (np.iinfo(np.uint32).max - 1) else np.uint32
    first = np.arange(0, num_samples, dtype=dtype_)
    np_rng.shuffle(first)
    if num_samples == total_size:
        return first
    last = np.arange(num_samples, total_size, dtype=dtype_)
    np_rng.shuffle(last)
    return np.concatenate((first, last))


def build_index_mappings(sizes, total_samples, seq_length, seed, cutoff_last_epoch=0.95):
    """(sentense_idx, location_idx, shuffle_idx) as `load_index_mappings` builds them (nlp_dataset.py:481-560), with the
    same consumption order of the seeded RandomState, so a cache built by either side indexes the same samples."""
    sizes = np.asarray(sizes, dtype=np.int32)
    sentenses_id = np.arange(sizes.shape[0], dtype=np.int32)
    tokens_per_epoch = int(np.sum(sizes[sentenses_id]))
    num_epochs = num_epochs_for(tokens_per_epoch, seq_length, total_samples)
    np_rng = np.random.RandomState(seed=seed)
    separate_last_epoch = False
    minus_one = 0
    if num_epochs > 1:
        minus_one = ((num_epochs - 1) * tokens_per_epoch - 1) // seq_length
        last_epoch = total_samples - minus_one
        per_epoch = (tokens_per_epoch - 1) // seq_length
        assert 0 <= last_epoch <= per_epoch, "last epoch number of samples %d outside [0, %d]" % (last_epoch, per_epoch)
        separate_last_epoch = last_epoch < int(cutoff_last_epoch * per_epoch)
    sentense_idx = build_sentense_idx(sentenses_id, num_epochs, np_rng, separate_last_epoch)
    location_idx = build_location_idx(sizes, sentense_idx, seq_length, num_epochs, tokens_per_epoch)
    num_samples_ = minus_one if separate_last_epoch else location_idx.shape[0] - 1
    shuffle_idx = build_shuffle_idx(num_samples_, location_idx.shape[0] - 1, np_rng)
    return sentense_idx, location_idx, shuffle_idx


class MMapIndexDataset(torch.utils.data.Dataset):
    """Samples of max_seq_length + 1 tokens cut from the concatenated, per-epoch shuffled documents of a token cache.

    Items are `{'input_ids', 'labels'}` (labels = input_ids, the shift happens in the batch function) plus, with
    `with_cu_lens`, `cu_seqlens` (document boundaries after each eos token) and `position_ids` restarting per document
    (nlp_dataset.py:585-636)."""

    def __init__(self, cache_prefix, seed, total_samples, max_seq_length, eos_token_id=None, cutoff_last_epoch=0.95,
                 with_cu_lens=False, shuffle=True):
        if not (os.path.exists(index_file_path(cache_prefix)) and os.path.exists(data_file_path(cache_prefix))):
            raise FileNotFoundError("no token cache %s.idx/.bin" % cache_prefix)
        if with_cu_lens and eos_token_id is None:
            raise ValueError("with_cu_lens needs the tokenizer's eos_token_id")
        self._index = MMapIndex(index_file_path(cache_prefix))
        self._bin = np.memmap(data_file_path(cache_prefix), mode="r", order="C")
        self.eos_token_id = eos_token_id
        self.with_cu_lens = with_cu_lens
        self.sentenses_idx, self.location_idx, self.shuffle_idx = build_index_mappings(
            self._index.sizes, total_samples, max_seq_length, seed, cutoff_last_epoch)
        if not shuffle:
            self.shuffle_idx = np.arange(self.location_idx.shape[0] - 1)

    def mmap_get_items(self, idx, offset=0, length=None):
        ptr, size = self._index[idx]
        if length is None:
            length = size - offset
        itemsize = np.dtype(self._index.dtype).itemsize
        return np.frombuffer(self._bin, dtype=self._index.dtype, count=int(length), offset=int(ptr) + int(offset) * itemsize)

    def __len__(self):
        return self.location_idx.shape[0] - 1

    def __getitem__(self, idx):
        idx = int(self.shuffle_idx[idx])
        doc_f, off_f = self.location_idx[idx]
        doc_l, off_l = self.location_idx[idx + 1]
        if doc_f == doc_l:
            sample = self.mmap_get_items(self.sentenses_idx[doc_f], offset=off_f, length=off_l - off_f + 1)
        else:
            parts = [self.mmap_get_items(self.sentenses_idx[doc_f], offset=off_f)]
            parts += [self.mmap_get_items(self.sentenses_idx[i]) for i in range(doc_f + 1, doc_l)]
            parts.append(self.mmap_get_items(self.sentenses_idx[doc_l], length=off_l + 1))
            sample = np.concatenate(parts)
        input_ids = torch.from_numpy(sample.astype(np.int64))
        results = {"input_ids": input_ids, "labels": input_ids.clone()}
        if self.with_cu_lens:
            cu = get_cu_seqlens(input_ids, self.eos_token_id)
            results.update({"cu_seqlens": torch.LongTensor(cu), "position_ids": torch.LongTensor(get_position_ids(cu))})
        return results


class MMapIndexJsonDataset(MMapIndexDataset):
    """The reference's `mmap_index_json` dataset (nlp_dataset.py:322-395): builds the token cache under
    `<data_root>/<cache_dir>/<cache_prefix>` from `json_file` when it does not exist yet, then serves packed samples from it.

    tokenizer: any object with `vocab_size` and `eos_token_id`.  transformer: a callable `meta -> {'input_ids': ...}` applied
    to each parsed json line (the reference builds it from its parser registry, which is outside this build); without one
    the lines must already hold `input_ids`.  Only the native sample-location builder exists, so `cache_location_builder`
    is accepted and ignored."""

    def __init__(self, data_root, seed, total_samples, max_seq_length, json_file=None, json_type="line", tokenizer=None,
                 transformer=None, cache_dir="train_data_cache", cache_prefix="mmap_sentebnse", cache_worker=4,
                 cache_skip_warmup=True, cache_log_freq=100, cache_splits=1, cache_location_builder="py", ignore_index=-100,
                 cutoff_last_epoch=0.95, with_cu_lens=False):
        self.tokenizer = tokenizer
        self.transformer = transformer
        self.ignore_index = ignore_index
        prefix = os.path.join(data_root, cache_dir, cache_prefix)
        if not (os.path.exists(index_file_path(prefix)) and os.path.exists(data_file_path(prefix))):
            os.makedirs(os.path.join(data_root, cache_dir), exist_ok=True)
            assert json_file is not None, ("you have not a cache .bin&.idx file of cache_prefix: {}, you must provide as least "
                                           "one json file to generate them".format(prefix))
            assert json_type == "line", "Only support line type json to build the cache .bin&.idx file"
            build_data_cache(self.data_encode, getattr(tokenizer, "vocab_size", None), json_file, prefix, cache_worker,
                             cache_splits=cache_splits)
        super().__init__(prefix, seed, total_samples, max_seq_length, eos_token_id=getattr(tokenizer, "eos_token_id", None),
                         cutoff_last_epoch=cutoff_last_epoch, with_cu_lens=with_cu_lens)

    def data_encode(self, json_line):
        if self.transformer is None:
            return encode_tokenised_line(json_line)
        return self.transformer(json.loads(json_line))
