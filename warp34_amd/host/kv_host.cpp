// Host side of the paged KV cache (see kv_host.h for the reference files each part mirrors).
#include "kv_host.h"

#include <algorithm>
#include <cstring>
#include <utility>

namespace warp34_host {

// ---- format policy ----------------------------------------------------------------------------
size_t kv_format_row_bytes(int format, size_t head_dim) {
    switch (format) {
        case WARP34_KV_FORMAT_FP16:
        case WARP34_KV_FORMAT_BF16: return head_dim * 2;
        case WARP34_KV_FORMAT_TQ4: return 66 * (head_dim / 128);        // fp16 scale + 64 code bytes per 128
        case WARP34_KV_FORMAT_Q8_0: return 68 * (head_dim / 64);        // f32 scale + 64 int8 per 64
        case WARP34_KV_FORMAT_FP8_E4M3: return head_dim + 4 * (head_dim / 128);
        default: return head_dim * 2;
    }
}

LayerFormats resolve_layer_with_fp8(KvFormatPolicy policy, size_t ordinal, size_t num_layers, bool supports_fp8_kv) {
    const int id = WARP34_KV_TRANSFORM_IDENTITY;
    const int wht = WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
    const LayerFormats tq4{WARP34_KV_FORMAT_TQ4, WARP34_KV_FORMAT_TQ4, wht, wht};
    switch (policy) {
        case KvFormatPolicy::Fp16: return {WARP34_KV_FORMAT_FP16, WARP34_KV_FORMAT_FP16, id, id};
        case KvFormatPolicy::Bf16: return {WARP34_KV_FORMAT_BF16, WARP34_KV_FORMAT_BF16, id, id};
        case KvFormatPolicy::Q8_0: return {WARP34_KV_FORMAT_Q8_0, WARP34_KV_FORMAT_Q8_0, id, id};
        case KvFormatPolicy::Fp8: return {WARP34_KV_FORMAT_FP8_E4M3, WARP34_KV_FORMAT_FP8_E4M3, id, id};
        case KvFormatPolicy::Tq4: {
            const size_t first_anchor = num_layers >= 4 ? num_layers - 4 : 0;
            if (ordinal >= first_anchor) {
                const int f = supports_fp8_kv ? WARP34_KV_FORMAT_FP8_E4M3 : WARP34_KV_FORMAT_Q8_0;
                return {f, f, id, id};
            }
            return tq4;
        }
        case KvFormatPolicy::Tq4All: return tq4;
    }
    return tq4;
}

size_t bytes_per_token_with_fp8(KvFormatPolicy policy, size_t num_layers, size_t kv_heads, size_t head_dim,
                                bool supports_fp8_kv) {
    size_t total = 0;
    for (size_t ord = 0; ord < num_layers; ++ord) {
        const LayerFormats f = resolve_layer_with_fp8(policy, ord, num_layers, supports_fp8_kv);
        total += kv_heads * (kv_format_row_bytes(f.k_format, head_dim) + kv_format_row_bytes(f.v_format, head_dim));
    }
    return total;
}

static const std::pair<const char*, KvFormatPolicy> kPolicyNames[] = {
    {"fp16", KvFormatPolicy::Fp16}, {"bf16", KvFormatPolicy::Bf16},     {"q8_0", KvFormatPolicy::Q8_0},
    {"fp8", KvFormatPolicy::Fp8},   {"tq4", KvFormatPolicy::Tq4},       {"tq4_all", KvFormatPolicy::Tq4All},
};

std::optional<KvFormatPolicy> parse_kv_policy(const std::string& name) {
    for (const auto& p : kPolicyNames)
        if (name == p.first) return p.second;
    return std::nullopt;
}

const char* kv_policy_name(KvFormatPolicy policy) {
    for (const auto& p : kPolicyNames)
        if (p.second == policy) return p.first;
    return "?";
}

// ---- page allocator ---------------------------------------------------------------------------
PageBitmap::PageBitmap(size_t num_pages)
    : num_pages_(num_pages), words_((num_pages + 63) / 64, 0), free_count_(0), next_word_(0) {
    reset();
}

void PageBitmap::reset() {
    const size_t full_words = num_pages_ / 64, rem = num_pages_ % 64;
    for (size_t w = 0; w < full_words; ++w) words_[w] = ~0ull;
    if (rem > 0) words_[full_words] = (1ull << rem) - 1;
    free_count_ = num_pages_;
    next_word_ = 0;
}

std::optional<int32_t> PageBitmap::alloc() {
    if (free_count_ == 0) return std::nullopt;
    const size_t n = words_.size();
    // from the cursor to the end, then the part before the cursor
    for (size_t step = 0; step < n; ++step) {
        const size_t w = next_word_ + step < n ? next_word_ + step : next_word_ + step - n;
        const uint64_t word = words_[w];
        if (word != 0) {
            const int bit = __builtin_ctzll(word);
            words_[w] = word & ~(1ull << bit);
            --free_count_;
            next_word_ = w;
            return (int32_t)(w * 64 + (size_t)bit);
        }
    }
    return std::nullopt;
}

void PageBitmap::free(int32_t page_id) {
    if (page_id < 0 || (size_t)page_id >= num_pages_) return;
    const size_t w = (size_t)page_id / 64;
    const uint64_t mask = 1ull << ((size_t)page_id % 64);
    if ((words_[w] & mask) == 0) {
        words_[w] |= mask;
        ++free_count_;
        if (w < next_word_) next_word_ = w;
    }
}

bool PageBitmap::is_free(int32_t page_id) const {
    if (page_id < 0 || (size_t)page_id >= num_pages_) return false;
    return (words_[(size_t)page_id / 64] >> ((size_t)page_id % 64)) & 1ull;
}

// ---- KV pool ----------------------------------------------------------------------------------
HostError KvPool::create(KvPool* out, DeviceAllocator& alloc, int device_id, int namespace_id,
                         const std::vector<size_t>& layer_ids, size_t local_kv_heads, size_t head_dim,
                         size_t block_size, size_t num_pages, KvFormatPolicy policy, bool supports_fp8_kv) {
    if (policy == KvFormatPolicy::Fp8 && !supports_fp8_kv)
        return HostError{-23, "unsupported KV format on GPU architecture: --kv-format fp8 needs hardware FP8"};
    KvPool pool;
    pool.alloc_ = &alloc;
    pool.device_id = device_id;
    pool.num_pages = num_pages;
    pool.block_size = block_size;
    const size_t num_full = layer_ids.size();
    for (size_t ord = 0; ord < num_full; ++ord) {
        const LayerFormats f = resolve_layer_with_fp8(policy, ord, num_full, supports_fp8_kv);
        const size_t k_tok = kv_format_row_bytes(f.k_format, head_dim);
        const size_t v_tok = kv_format_row_bytes(f.v_format, head_dim);
        const size_t k_head = block_size * k_tok, v_head = block_size * v_tok;
        const size_t k_page = local_kv_heads * k_head, v_page = local_kv_heads * v_head;
        KvLayerBuffer lb;
        lb.k_bytes = num_pages * k_page;
        lb.v_bytes = num_pages * v_page;
        int rc = alloc.alloc(device_id, lb.k_bytes, &lb.k_buf);
        if (rc == 0) {
            rc = alloc.alloc(device_id, lb.v_bytes, &lb.v_buf);
            if (rc != 0) alloc.release(device_id, lb.k_buf);
        }
        if (rc != 0) return HostError{rc, "KV slab allocation failed for layer " + std::to_string(layer_ids[ord])};
        warp34_kv_layer_layout& L = lb.layout;
        L.k_base = lb.k_buf;
        L.v_base = lb.v_buf;
        L.k_page_stride_bytes = k_page;
        L.k_head_stride_bytes = k_head;
        L.k_token_stride_bytes = k_tok;
        L.v_page_stride_bytes = v_page;
        L.v_head_stride_bytes = v_head;
        L.v_token_stride_bytes = v_tok;
        L.namespace_id = namespace_id;
        L.layer_id = (int32_t)layer_ids[ord];
        L.local_kv_heads = (int32_t)local_kv_heads;
        L.head_dim = (int32_t)head_dim;
        L.block_size = (int32_t)block_size;
        L.k_format = f.k_format;
        L.v_format = f.v_format;
        L.k_transform = f.k_transform;
        L.v_transform = f.v_transform;
        L.reserved = 0;
        pool.layers.push_back(lb);
    }
    pool.free_pages_ = PageBitmap(num_pages);
    *out = std::move(pool);
    return HostError{};
}

void KvPool::release() {
    if (alloc_ != nullptr)
        for (KvLayerBuffer& lb : layers) {
            if (lb.k_buf) alloc_->release(device_id, lb.k_buf);
            if (lb.v_buf) alloc_->release(device_id, lb.v_buf);
        }
    layers.clear();
}

KvPool::~KvPool() { release(); }

KvPool::KvPool(KvPool&& o) noexcept : free_pages_(0) { *this = std::move(o); }

KvPool& KvPool::operator=(KvPool&& o) noexcept {
    if (this != &o) {
        release();
        device_id = o.device_id;
        num_pages = o.num_pages;
        block_size = o.block_size;
        layers = std::move(o.layers);
        o.layers.clear();
        alloc_ = o.alloc_;
        free_pages_ = o.free_pages_;
    }
    return *this;
}

void KvPool::truncate_pages(size_t max_pages) {
    if (max_pages < num_pages) {
        num_pages = max_pages;
        free_pages_ = PageBitmap(max_pages);
    }
}

// ---- slot mapping and the packed step descriptor ----------------------------------------------
std::vector<int32_t> write_slot_mapping(const std::vector<int32_t>& block_table, size_t ctx_before,
                                        size_t seq_after, size_t block_size) {
    std::vector<int32_t> slots;
    slots.reserve(seq_after > ctx_before ? seq_after - ctx_before : 0);
    for (size_t pos = ctx_before; pos < seq_after; ++pos)
        slots.push_back(block_table[pos / block_size] * (int32_t)block_size + (int32_t)(pos % block_size));
    return slots;
}

StepMeta pack_step_meta(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                        const std::vector<int32_t>& block_table, size_t ctx_before, size_t seq_after,
                        size_t block_size, int32_t state_in_slot, int32_t state_out_slot, bool has_initial_state) {
    StepMeta m;
    const std::vector<int32_t> slots = write_slot_mapping(block_table, ctx_before, seq_after, block_size);
    m.tok_words = tokens.size();
    m.pos_words = positions.size();
    m.slot_words = slots.size();
    m.blk_words = block_table.size();
    m.ctx_before = ctx_before;
    m.seq_after = seq_after;
    m.words.reserve(m.tok_words + m.pos_words + m.slot_words + m.blk_words + 7);
    m.words.insert(m.words.end(), tokens.begin(), tokens.end());
    m.words.insert(m.words.end(), positions.begin(), positions.end());
    m.words.insert(m.words.end(), slots.begin(), slots.end());
    m.words.insert(m.words.end(), block_table.begin(), block_table.end());
    const int32_t tail[7] = {0, (int32_t)tokens.size(), (int32_t)ctx_before, (int32_t)seq_after,
                             state_in_slot, state_out_slot, has_initial_state ? 1 : 0};
    m.words.insert(m.words.end(), tail, tail + 7);
    return m;
}

warp34_attention_batch StepMeta::batch_at(uint64_t dev_base, int mask_mode, float sm_scale) const {
    const uint64_t slot_ptr = dev_base + 4 * (tok_words + pos_words);
    const uint64_t blk_ptr = slot_ptr + 4 * slot_words;
    const uint64_t q_start_ptr = blk_ptr + 4 * blk_words;
    warp34_attention_batch b;
    std::memset(&b, 0, sizeof b);
    b.query_start_loc = (const int32_t*)(uintptr_t)q_start_ptr;
    b.context_lens_before = (const int32_t*)(uintptr_t)(q_start_ptr + 8);
    b.seq_lens_after = (const int32_t*)(uintptr_t)(q_start_ptr + 12);
    b.block_tables = (const int32_t*)(uintptr_t)blk_ptr;
    b.write_slot_mapping = (const int32_t*)(uintptr_t)slot_ptr;
    b.valid_token_mask = nullptr;
    b.valid_req_mask = nullptr;
    b.num_reqs = 1;
    b.total_tokens = (int32_t)tok_words;
    b.max_blocks_per_req = (int32_t)blk_words;
    b.max_q_len = (int32_t)tok_words;
    b.max_seq_len = (int32_t)seq_after;
    b.mask_mode = mask_mode;
    b.sliding_window = 0;
    b.sm_scale = sm_scale;
    b.reserved = 0;
    return b;
}

// ---- page reservation (model/batch.rs:57-103); the prefix tree itself lives in prefix_cache.cpp ----
bool reserve_kv_pages_from(KvPool& pool, PrefixPageCache& cache, std::vector<int32_t>* dst, size_t target_pages) {
    if (dst->size() >= target_pages) return true;
    const size_t missing = target_pages - dst->size();
    const size_t avail = pool.free_count();
    if (avail < missing) {
        const EvictResult ev = cache.evict_full_pages(missing - avail);
        free_kv_pages(pool, ev.freed_kv_pages);
    }
    if (pool.free_count() < missing) return false;
    dst->reserve(target_pages);
    for (size_t i = 0; i < missing; ++i) dst->push_back(*pool.alloc_page());
    return true;
}

void free_kv_pages(KvPool& pool, const std::vector<int32_t>& pages) {
    for (int32_t p : pages)
        if (p >= 0) pool.free_page(p);
}

}  // namespace warp34_host
