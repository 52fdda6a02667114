// Host-side index builder for packed-sequence datasets (no GPU code).
//
// Replaces the reference's only native component, `build_location_idx` of llm/data/cores/helpers.cpp:36-122 (bound
// with pybind11 there; python twin at llm/data/nlp_dataset.py:424-463): documents, taken in the order given by
// `doc_idx`, are laid end to end and cut into samples of seq_length + 1 tokens that overlap by one token; row k of the
// result is (position in doc_idx, token offset inside that document) of the first token of sample k.
//
// Formulated through the running token position instead of the reference's remaining-length countdown: sample k starts
// at global token k * seq_length, so one forward sweep over the documents places every row.  Zero-length documents are
// skipped, and a boundary that coincides with a document's last token stays on that token, as in the reference.
// Unlike the reference, which reads past its arrays on inconsistent input, every access is bounds-checked.
#include "common.h"

extern "C" int64_t ezl_location_idx_rows(int64_t seq_length, int64_t num_epochs, int64_t tokens_per_epoch) {
    if (seq_length <= 1 || num_epochs <= 0 || tokens_per_epoch <= 1) return -1;
    return (num_epochs * tokens_per_epoch - 1) / seq_length + 1;
}

extern "C" int ezl_build_location_idx(const int32_t* sizes, int64_t n_sizes, const int32_t* doc_idx, int64_t n_doc_idx,
                                      int64_t seq_length, int64_t num_epochs, int64_t tokens_per_epoch, int32_t* out,
                                      int64_t out_rows) {
    const int64_t rows = ezl_location_idx_rows(seq_length, num_epochs, tokens_per_epoch);
    EZL_REQUIRE(rows > 0, EZL_EINVAL, "ezl_build_location_idx: need seq_length > 1, num_epochs > 0, tokens_per_epoch > 1");
    EZL_REQUIRE(sizes && doc_idx && out && n_sizes > 0 && n_doc_idx > 0, EZL_EINVAL, "ezl_build_location_idx: null or empty input");
    EZL_REQUIRE(out_rows == rows, EZL_EINVAL, "ezl_build_location_idx: output must have %lld rows", (long long)rows);
    int64_t d = 0;        // position in doc_idx
    int64_t before = 0;   // tokens in documents before position d
    for (int64_t k = 0; k < rows; ++k) {
        const int64_t target = k * seq_length;  // global index of the sample's first token
        for (;;) {
            EZL_REQUIRE(d < n_doc_idx, EZL_EINVAL,
                        "ezl_build_location_idx: the documents hold fewer than num_epochs * tokens_per_epoch tokens");
            const int32_t doc = doc_idx[d];
            EZL_REQUIRE(doc >= 0 && doc < n_sizes, EZL_EINVAL, "ezl_build_location_idx: document id %d out of range", (int)doc);
            const int64_t len = sizes[doc];
            EZL_REQUIRE(len >= 0, EZL_EINVAL, "ezl_build_location_idx: negative document size");
            if (target < before + len) break;
            before += len;
            ++d;
        }
        EZL_REQUIRE(d <= 0x7fffffffLL, EZL_EUNSUPPORTED, "ezl_build_location_idx: more than 2^31 documents");
        out[2 * k] = (int32_t)d;
        out[2 * k + 1] = (int32_t)(target - before);
    }
    return EZL_OK;
}
