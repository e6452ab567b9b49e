// Fixed-shape step descriptors for captured (HIP graph) decode and speculative-verify steps:
// the host packs one small blob of i32 words (+ mask bytes), copies it over the blob the graph's
// kernels read, and replays.  Layouts and rules follow crates/warp34-host/src/model/graph_io.rs
// (DecodeGraph bucket table :585-595, BatchedDecodeGraphIo :647-871 and its block-table upload
// :886-1010, SpecVerifyGraphIo :285-421); the page size is a parameter here (the reference
// hard-codes 16 tokens).  Only the words the KV path reads are interpreted; token ids, state
// and adapter slots travel in the same blob because the reference's graphs read them from it.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <optional>
#include <utility>
#include <vector>

#include "../../include/warp34_kv.h"

namespace warp34_host {

constexpr int32_t kBaseModelLoraId = -1;

// One request's share of a step (EngineBatchSlice, model/execution.rs).
struct StepSlice {
    std::vector<int32_t> tokens;
    size_t ctx_len_before = 0;
    std::vector<int32_t> block_table;
    int32_t state_in_slot = -1, state_out_slot = -1;
    bool has_initial_state = false;
    std::vector<int32_t> spec_slots;
    std::vector<std::pair<int32_t, int32_t>> checkpoints;  // (1-based trigger offset, destination slot)
};

// ---- batched one-token decode (graph_io.rs:579-871) ---------------------------------------------
constexpr size_t kMaxBatchedDecodeReqs = 16;
// The captured graph a batch of num_reqs requests replays: 1, 2, 4, 8 or 16 rows; none beyond 16.
std::optional<size_t> decode_graph_bucket(size_t num_reqs);

struct BatchedDecodeMeta {
    static constexpr size_t N = kMaxBatchedDecodeReqs;
    static constexpr size_t kWords = 11 * N + 1;
    static constexpr size_t kMaskBytes = 3 * N;
    // word offsets
    static constexpr size_t kTokenIds = 0, kPositions = N, kWriteSlots = 2 * N, kQStartLoc = 3 * N,
                            kCtxBefore = 4 * N + 1, kSeqAfter = 5 * N + 1, kStateIn = 6 * N + 1, kStateOut = 7 * N + 1,
                            kCheckpointDst = 8 * N + 1, kCheckpointOffset = 9 * N + 1, kLoraIds = 10 * N + 1;
    // the masks follow the words at the next multiple of 64 bytes
    static constexpr size_t kMasksByteOffset = (kWords * 4 + 63) & ~size_t(63);
    static constexpr size_t kHasInitialState = 0, kValidReq = N, kValidToken = 2 * N;  // byte offsets inside the masks
    static constexpr size_t kBlobBytes = kMasksByteOffset + kMaskBytes;

    std::array<int32_t, kWords> words{};
    std::array<uint8_t, kMaskBytes> masks{};
    // The whole blob as it lies on the device (words, padding, masks): one host-to-device copy.
    std::array<uint8_t, kBlobBytes> blob() const;
    // The attention descriptor of a replay with `bucket` rows whose blob lies at dev_blob and whose
    // block tables ([kMaxBatchedDecodeReqs][max_blocks_per_req]) at dev_block_tables.  Rows
    // beyond the live requests are masked out by valid_req_mask / valid_token_mask and have
    // write slot -1.  max_seq_len is the host's bound for the bucket's captured launch.
    static warp34_attention_batch batch_at(uint64_t dev_blob, uint64_t dev_block_tables, size_t bucket,
                                           size_t max_blocks_per_req, size_t max_seq_len, int mask_mode,
                                           float sm_scale);
};
// false: no or too many slices, or a slice that is not a one-token decode step with enough pages
// (graph_io.rs:804-871).  rope_pos_deltas may be empty.
bool pack_batched_decode_meta(const std::vector<StepSlice>& slices, const std::vector<int32_t>& rope_pos_deltas,
                              const std::vector<int32_t>& slice_lora_ids, int32_t default_lora_id, size_t page_size,
                              BatchedDecodeMeta* out);

// What the device copy of the block tables holds, row by row, so that a step uploads only what
// changed: nothing for an unchanged row, the new tail for a row that grew, the whole row
// otherwise (graph_io.rs:886-1010).
struct BlockTableSpan {
    size_t row = 0, start = 0;      // first changed entry
    std::vector<int32_t> entries;   // the entries from there on
    size_t dst_byte_offset = 0;     // into the device array of rows of max_blocks_per_req entries
};
class BlockTableMirror {
public:
    explicit BlockTableMirror(size_t max_blocks_per_req);
    size_t max_blocks_per_req() const { return max_blocks_; }
    // spans to copy for this step, or nullopt when a row does not fit; the mirror is updated
    // (commit == true) as if the copies had been made
    std::optional<std::vector<BlockTableSpan>> dirty_spans(const std::vector<StepSlice>& slices, bool commit = true);
    // a failed copy: forget what the device is believed to hold for these rows
    void invalidate(const std::vector<BlockTableSpan>& spans);
    void invalidate_all();

private:
    size_t max_blocks_;
    std::vector<std::vector<int32_t>> rows_;
};

// ---- speculative verify of one request, 2..16 query tokens (graph_io.rs:285-421) ------------------
constexpr size_t kMaxSpecVerifyTokens = 16;
constexpr size_t kMaxSpecVerifyCheckpoints = 4;
struct SpecVerifyMeta {
    static constexpr size_t T = kMaxSpecVerifyTokens, CP = kMaxSpecVerifyCheckpoints;
    static constexpr size_t kWords = 5 * T + 2 * CP + 6;
    static constexpr size_t kTokenIds = 0, kPositions = T, kWriteSlots = 2 * T, kSpecSlots = 3 * T, kCheckpointDst = 4 * T,
                            kCheckpointOffset = 4 * T + CP, kQStartLoc = 4 * T + 2 * CP /* 2 words */,
                            kCtxBefore = kQStartLoc + 2, kSeqAfter = kQStartLoc + 3, kStateIn = kQStartLoc + 4,
                            kStateOut = kQStartLoc + 5, kLoraIds = kQStartLoc + 6;
    std::array<int32_t, kWords> words{};
    static warp34_attention_batch batch_at(uint64_t dev_words, uint64_t dev_block_table, size_t q_len,
                                           size_t max_blocks_per_req, size_t max_seq_len, int mask_mode, float sm_scale);
};
bool pack_spec_verify_meta(const StepSlice& slice, int32_t lora_id, size_t page_size, SpecVerifyMeta* out);

}  // namespace warp34_host
