// Step descriptors for captured decode / verify steps; see graph_io.h.
#include "graph_io.h"

#include <cstring>
#include <limits>

namespace warp34_host {

std::optional<size_t> decode_graph_bucket(size_t num_reqs) {
    if (num_reqs == 0 || num_reqs > kMaxBatchedDecodeReqs) return std::nullopt;
    size_t b = 1;
    while (b < num_reqs) b <<= 1;
    return b;
}

std::array<uint8_t, BatchedDecodeMeta::kBlobBytes> BatchedDecodeMeta::blob() const {
    std::array<uint8_t, kBlobBytes> b{};
    std::memcpy(b.data(), words.data(), kWords * 4);
    std::memcpy(b.data() + kMasksByteOffset, masks.data(), kMaskBytes);
    return b;
}

warp34_attention_batch BatchedDecodeMeta::batch_at(uint64_t dev_blob, uint64_t dev_block_tables, size_t bucket,
                                                   size_t max_blocks_per_req, size_t max_seq_len, int mask_mode,
                                                   float sm_scale) {
    warp34_attention_batch b{};
    auto word = [&](size_t off) { return reinterpret_cast<const int32_t*>((uintptr_t)(dev_blob + 4 * off)); };
    auto mask = [&](size_t off) { return reinterpret_cast<const uint8_t*>((uintptr_t)(dev_blob + kMasksByteOffset + off)); };
    b.query_start_loc = word(kQStartLoc);
    b.context_lens_before = word(kCtxBefore);
    b.seq_lens_after = word(kSeqAfter);
    b.block_tables = reinterpret_cast<const int32_t*>((uintptr_t)dev_block_tables);
    b.write_slot_mapping = word(kWriteSlots);
    b.valid_token_mask = mask(kValidToken);
    b.valid_req_mask = mask(kValidReq);
    b.num_reqs = (int32_t)bucket;
    b.total_tokens = (int32_t)bucket;
    b.max_blocks_per_req = (int32_t)max_blocks_per_req;
    b.max_q_len = 1;
    b.max_seq_len = (int32_t)max_seq_len;
    b.mask_mode = mask_mode;
    b.sliding_window = 0;
    b.sm_scale = sm_scale;
    b.reserved = 0;
    return b;
}

bool pack_batched_decode_meta(const std::vector<StepSlice>& slices, const std::vector<int32_t>& rope_pos_deltas,
                              const std::vector<int32_t>& slice_lora_ids, int32_t default_lora_id, size_t page_size,
                              BatchedDecodeMeta* out) {
    using M = BatchedDecodeMeta;
    const size_t n = slices.size();
    if (n == 0 || n > M::N || page_size == 0) return false;
    M m;
    for (size_t i = 0; i <= M::N; ++i) m.words[M::kQStartLoc + i] = (int32_t)i;  // one token per row, padding rows too
    for (size_t r = 0; r < M::N; ++r) {
        m.words[M::kWriteSlots + r] = -1;
        m.words[M::kStateOut + r] = -1;
        m.words[M::kCheckpointDst + r] = -1;
        m.words[M::kCheckpointOffset + r] = -1;
        m.words[M::kLoraIds + r] = kBaseModelLoraId;
    }
    for (size_t r = 0; r < n; ++r) {
        const StepSlice& s = slices[r];
        const size_t pos = s.ctx_len_before;
        if (s.tokens.size() != 1 || !s.spec_slots.empty() || s.checkpoints.size() > 1 ||
            pos >= (size_t)std::numeric_limits<int32_t>::max() ||
            s.block_table.size() < (pos + 1 + page_size - 1) / page_size) {
            return false;
        }
        const int32_t delta = r < rope_pos_deltas.size() ? rope_pos_deltas[r] : 0;
        m.words[M::kTokenIds + r] = s.tokens[0];
        m.words[M::kPositions + r] = (int32_t)pos + delta;
        m.words[M::kWriteSlots + r] = s.block_table[pos / page_size] * (int32_t)page_size + (int32_t)(pos % page_size);
        m.words[M::kCtxBefore + r] = (int32_t)pos;
        m.words[M::kSeqAfter + r] = (int32_t)pos + 1;
        m.words[M::kStateIn + r] = s.state_in_slot;
        m.words[M::kStateOut + r] = s.state_out_slot;
        if (!s.checkpoints.empty()) {
            m.words[M::kCheckpointDst + r] = s.checkpoints[0].second;
            m.words[M::kCheckpointOffset + r] = s.checkpoints[0].first;
        }
        m.words[M::kLoraIds + r] = r < slice_lora_ids.size() ? slice_lora_ids[r] : default_lora_id;
        m.masks[M::kHasInitialState + r] = s.has_initial_state ? 1 : 0;
        m.masks[M::kValidReq + r] = 1;
        m.masks[M::kValidToken + r] = 1;
    }
    *out = m;
    return true;
}

BlockTableMirror::BlockTableMirror(size_t max_blocks_per_req)
    : max_blocks_(max_blocks_per_req ? max_blocks_per_req : 1), rows_(kMaxBatchedDecodeReqs) {}

std::optional<std::vector<BlockTableSpan>> BlockTableMirror::dirty_spans(const std::vector<StepSlice>& slices,
                                                                         bool commit) {
    if (slices.size() > kMaxBatchedDecodeReqs) return std::nullopt;
    for (const StepSlice& s : slices)
        if (s.block_table.size() > max_blocks_) return std::nullopt;
    std::vector<BlockTableSpan> spans;
    for (size_t r = 0; r < slices.size(); ++r) {
        const std::vector<int32_t>& want = slices[r].block_table;
        const std::vector<int32_t>& have = rows_[r];
        if (have == want) continue;
        size_t start = 0;
        if (want.size() >= have.size() && std::equal(have.begin(), have.end(), want.begin())) start = have.size();
        if (start < want.size()) {
            BlockTableSpan sp;
            sp.row = r;
            sp.start = start;
            sp.entries.assign(want.begin() + (long)start, want.end());
            sp.dst_byte_offset = (r * max_blocks_ + start) * 4;
            spans.push_back(std::move(sp));
        }
        if (commit) rows_[r] = want;  // (a row that only shrank needs no copy: the entries behind its end are not read)
    }
    return spans;
}

void BlockTableMirror::invalidate(const std::vector<BlockTableSpan>& spans) {
    for (const BlockTableSpan& sp : spans)
        if (sp.row < rows_.size()) rows_[sp.row].clear();
}

void BlockTableMirror::invalidate_all() {
    for (auto& r : rows_) r.clear();
}

warp34_attention_batch SpecVerifyMeta::batch_at(uint64_t dev_words, uint64_t dev_block_table, size_t q_len,
                                                size_t max_blocks_per_req, size_t max_seq_len, int mask_mode,
                                                float sm_scale) {
    warp34_attention_batch b{};
    auto word = [&](size_t off) { return reinterpret_cast<const int32_t*>((uintptr_t)(dev_words + 4 * off)); };
    b.query_start_loc = word(kQStartLoc);
    b.context_lens_before = word(kCtxBefore);
    b.seq_lens_after = word(kSeqAfter);
    b.block_tables = reinterpret_cast<const int32_t*>((uintptr_t)dev_block_table);
    b.write_slot_mapping = word(kWriteSlots);
    b.valid_token_mask = nullptr;
    b.valid_req_mask = nullptr;
    b.num_reqs = 1;
    b.total_tokens = (int32_t)q_len;
    b.max_blocks_per_req = (int32_t)max_blocks_per_req;
    b.max_q_len = (int32_t)q_len;
    b.max_seq_len = (int32_t)max_seq_len;
    b.mask_mode = mask_mode;
    b.sliding_window = 0;
    b.sm_scale = sm_scale;
    b.reserved = 0;
    return b;
}

bool pack_spec_verify_meta(const StepSlice& s, int32_t lora_id, size_t page_size, SpecVerifyMeta* out) {
    using M = SpecVerifyMeta;
    const size_t q_len = s.tokens.size();
    if (page_size == 0 || s.ctx_len_before > (size_t)std::numeric_limits<int32_t>::max() - M::T) return false;
    const size_t seq_after = s.ctx_len_before + q_len;
    if (q_len == 0 || q_len > M::T || s.spec_slots.size() > M::T || s.checkpoints.size() > M::CP ||
        s.block_table.size() < (seq_after + page_size - 1) / page_size) {
        return false;
    }
    M m;
    m.words.fill(-1);
    for (size_t step = 0; step < q_len; ++step) {
        const size_t pos = s.ctx_len_before + step;
        m.words[M::kTokenIds + step] = s.tokens[step];
        m.words[M::kPositions + step] = (int32_t)pos;
        m.words[M::kWriteSlots + step] = s.block_table[pos / page_size] * (int32_t)page_size + (int32_t)(pos % page_size);
        m.words[M::kLoraIds + step] = lora_id;
    }
    for (size_t i = 0; i < s.spec_slots.size(); ++i) m.words[M::kSpecSlots + i] = s.spec_slots[i];
    for (size_t e = 0; e < s.checkpoints.size(); ++e) {
        m.words[M::kCheckpointDst + e] = s.checkpoints[e].second;
        m.words[M::kCheckpointOffset + e] = s.checkpoints[e].first;
    }
    m.words[M::kQStartLoc] = 0;
    m.words[M::kQStartLoc + 1] = (int32_t)q_len;
    m.words[M::kCtxBefore] = (int32_t)s.ctx_len_before;
    m.words[M::kSeqAfter] = (int32_t)seq_after;
    m.words[M::kStateIn] = s.state_in_slot;
    m.words[M::kStateOut] = s.state_out_slot;
    *out = m;
    return true;
}

}  // namespace warp34_host

// ---- C ABI (include/warp34_host.h) ----------------------------------------------------------------
#include "../../include/warp34_host.h"

static_assert(WARP34_HOST_DECODE_BLOB_BYTES == warp34_host::BatchedDecodeMeta::kBlobBytes, "blob size");
static_assert(WARP34_HOST_MAX_BATCHED_DECODE_REQS == warp34_host::kMaxBatchedDecodeReqs, "rows");

extern "C" int warp34_host_decode_graph_bucket(int num_reqs) {
    if (num_reqs <= 0) return 0;
    const auto b = warp34_host::decode_graph_bucket((size_t)num_reqs);
    return b ? (int)*b : 0;
}

extern "C" int warp34_host_pack_batched_decode_blob(const int32_t* tokens, const int32_t* ctx_lens_before,
                                                    const int32_t* block_tables, const int32_t* block_table_lens,
                                                    int bt_stride, int num_reqs, int page_size, uint8_t* blob_out) {
    if (!tokens || !ctx_lens_before || !block_tables || !block_table_lens || !blob_out || num_reqs <= 0 ||
        num_reqs > WARP34_HOST_MAX_BATCHED_DECODE_REQS || bt_stride <= 0 || page_size <= 0) {
        return 1;
    }
    std::vector<warp34_host::StepSlice> slices((size_t)num_reqs);
    for (int r = 0; r < num_reqs; ++r) {
        if (ctx_lens_before[r] < 0 || block_table_lens[r] < 0 || block_table_lens[r] > bt_stride) return 1;
        slices[r].tokens = {tokens[r]};
        slices[r].ctx_len_before = (size_t)ctx_lens_before[r];
        slices[r].block_table.assign(block_tables + (size_t)r * bt_stride,
                                     block_tables + (size_t)r * bt_stride + block_table_lens[r]);
    }
    warp34_host::BatchedDecodeMeta m;
    if (!warp34_host::pack_batched_decode_meta(slices, {}, {}, warp34_host::kBaseModelLoraId, (size_t)page_size, &m)) return 1;
    const auto blob = m.blob();
    std::memcpy(blob_out, blob.data(), blob.size());
    return 0;
}

extern "C" void warp34_host_batched_decode_batch_at(uint64_t dev_blob, uint64_t dev_block_tables, int bucket,
                                                    int max_blocks_per_req, int max_seq_len, int mask_mode,
                                                    float sm_scale, warp34_attention_batch* out) {
    *out = warp34_host::BatchedDecodeMeta::batch_at(dev_blob, dev_block_tables, (size_t)bucket, (size_t)max_blocks_per_req,
                                                    (size_t)max_seq_len, mask_mode, sm_scale);
}
