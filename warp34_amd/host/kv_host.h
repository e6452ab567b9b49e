// Host side of the paged KV cache: format policy, page allocator, KV pool descriptors,
// slot mapping, step-descriptor packing, page reservation and prefix-shared pages.
//
// C++ mirror of the reference's Rust operators for this path; names, argument meaning and
// error behaviour follow
//   crates/warp34-host/src/cache.rs:27-165   KvFormatPolicy, kv_format_row_bytes
//   crates/warp34-host/src/cache.rs:178-264  PageBitmap
//   crates/warp34-host/src/cache.rs:266-416  KvPool
//   crates/warp34-host/src/model/execution.rs:7-143,382-388  slot mapping, packed step blob
//   crates/warp34-host/src/model/batch.rs:27-103             page reservation
//   crates/warp34-host/src/radix.rs:383-490,1129-1157,1234-1245  prefix hit, rollback
// so that a Rust binding over the same C ABI is mechanical.  Nothing here touches the GPU
// except through the DeviceAllocator handed to KvPool.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/warp34_kv.h"

namespace warp34_host {

// ---- format policy (cache.rs:27-165) ----------------------------------------------------------
enum class KvFormatPolicy { Fp16, Bf16, Q8_0, Fp8, Tq4, Tq4All };

struct LayerFormats {
    int k_format, v_format, k_transform, v_transform;
    bool operator==(const LayerFormats& o) const {
        return k_format == o.k_format && v_format == o.v_format && k_transform == o.k_transform &&
               v_transform == o.v_transform;
    }
};

// Row bytes of one head in `format`; unknown formats size like 16-bit rows (cache.rs:157-165).
size_t kv_format_row_bytes(int format, size_t head_dim);

// What DeviceProps::supports_fp8_kv() (model/rank.rs:924-932) answers for the device these kernels
// are written for: gfx950 converts OCP E4M3 in hardware and the FP8 append and attention
// kernels are built, so the Tq4 policy's tail layers resolve to FP8.
constexpr bool kDeviceSupportsFp8Kv = true;

// Tq4: the last four full-attention layers are unrotated 8-bit (FP8 when the device has it,
// else Q8_0), all earlier ones rotated TQ4 (cache.rs:87-109).
LayerFormats resolve_layer_with_fp8(KvFormatPolicy policy, size_t full_attn_layer_ordinal,
                                    size_t num_full_attn_layers, bool supports_fp8_kv);
inline LayerFormats resolve_layer(KvFormatPolicy policy, size_t ordinal, size_t num_layers) {
    return resolve_layer_with_fp8(policy, ordinal, num_layers, false);
}
size_t bytes_per_token_with_fp8(KvFormatPolicy policy, size_t num_full_attn_layers, size_t kv_heads,
                                size_t head_dim, bool supports_fp8_kv);
inline size_t bytes_per_token(KvFormatPolicy policy, size_t num_layers, size_t kv_heads, size_t head_dim) {
    return bytes_per_token_with_fp8(policy, num_layers, kv_heads, head_dim, false);
}
// "fp16" | "bf16" | "q8_0" | "fp8" | "tq4" | "tq4_all" (the --kv-format spellings)
std::optional<KvFormatPolicy> parse_kv_policy(const std::string& name);
const char* kv_policy_name(KvFormatPolicy policy);

// ---- page allocator (cache.rs:178-264) --------------------------------------------------------
// Free-page bitmap that always hands out the lowest free page id; `next_word` is a scan cursor
// that a free below it pulls back.  Duplicate and out-of-range frees are ignored.
class PageBitmap {
public:
    explicit PageBitmap(size_t num_pages);
    size_t free_count() const { return free_count_; }
    size_t num_pages() const { return num_pages_; }
    void reset();
    std::optional<int32_t> alloc();
    void free(int32_t page_id);
    bool is_free(int32_t page_id) const;

private:
    size_t num_pages_;
    std::vector<uint64_t> words_;
    size_t free_count_;
    size_t next_word_;
};

// ---- KV pool (cache.rs:266-416) ---------------------------------------------------------------
struct DeviceAllocator {
    virtual ~DeviceAllocator() = default;
    virtual int alloc(int device_id, size_t bytes, uint64_t* addr) = 0;  // 0 on success
    virtual void release(int device_id, uint64_t addr) = 0;
};
// warp34_malloc / warp34_free of the kernel library (resolved at link time by the caller).
DeviceAllocator& runtime_allocator();

struct KvLayerBuffer {
    uint64_t k_buf = 0, v_buf = 0;
    size_t k_bytes = 0, v_bytes = 0;
    warp34_kv_layer_layout layout{};
};

struct HostError {
    int code = 0;  // 0 ok; positive = HIP error of the allocator; negative = host-synthetic
    std::string detail;
    explicit operator bool() const { return code != 0; }
};

class KvPool {
public:
    // One K and one V slab per full-attention layer; strides: token = row bytes,
    // head = block_size * token, page = local_kv_heads * head (cache.rs:304-335).
    // Fp8 policy on a device without FP8 KV support fails with code -23 (cache.rs:289-301).
    static HostError create(KvPool* out, DeviceAllocator& alloc, int device_id, int namespace_id,
                            const std::vector<size_t>& layer_ids, size_t local_kv_heads, size_t head_dim,
                            size_t block_size, size_t num_pages, KvFormatPolicy policy, bool supports_fp8_kv);
    static HostError new_target_full_attn(KvPool* out, DeviceAllocator& alloc, int device_id,
                                          const std::vector<size_t>& layer_ids, size_t local_kv_heads,
                                          size_t head_dim, size_t block_size, size_t num_pages,
                                          KvFormatPolicy policy, bool supports_fp8_kv) {
        return create(out, alloc, device_id, WARP34_KV_NAMESPACE_TARGET_FULL_ATTN, layer_ids, local_kv_heads,
                      head_dim, block_size, num_pages, policy, supports_fp8_kv);
    }
    KvPool() : free_pages_(0) {}
    ~KvPool();
    KvPool(const KvPool&) = delete;
    KvPool& operator=(const KvPool&) = delete;
    KvPool(KvPool&& o) noexcept;
    KvPool& operator=(KvPool&& o) noexcept;

    size_t free_count() const { return free_pages_.free_count(); }
    std::optional<int32_t> alloc_page() { return free_pages_.alloc(); }
    void free_page(int32_t page_id) { free_pages_.free(page_id); }
    void reset_all_pages() { free_pages_.reset(); }
    // Lowers the logical capacity (never raises it) and resets the free list (cache.rs:409-414).
    void truncate_pages(size_t max_pages);

    int device_id = 0;
    size_t num_pages = 0;
    size_t block_size = 0;
    std::vector<KvLayerBuffer> layers;

private:
    void release();
    DeviceAllocator* alloc_ = nullptr;
    PageBitmap free_pages_;
};

// ---- slot mapping and the packed step descriptor (execution.rs:7-143,382-388) -----------------
// slot(pos) = block_table[pos / block_size] * block_size + pos % block_size for pos in
// [ctx_before, seq_after).
std::vector<int32_t> write_slot_mapping(const std::vector<int32_t>& block_table, size_t ctx_before,
                                        size_t seq_after, size_t block_size);

// One request's step metadata as ONE host blob of i32 words, uploaded with a single H2D copy:
//   tokens | positions | write slots | block table | 0, N, ctx_before, seq_after, state_in,
//   state_out, has_initial_state
// `batch_at(dev_base)` yields the attention descriptor whose device pointers index into the
// uploaded copy at dev_base.
struct StepMeta {
    std::vector<int32_t> words;
    size_t tok_words = 0, pos_words = 0, slot_words = 0, blk_words = 0;
    size_t ctx_before = 0, seq_after = 0;
    size_t bytes() const { return words.size() * 4; }
    uint64_t tokens_at(uint64_t dev_base) const { return dev_base; }
    uint64_t positions_at(uint64_t dev_base) const { return dev_base + 4 * tok_words; }
    warp34_attention_batch batch_at(uint64_t dev_base, int mask_mode, float sm_scale) const;
};
StepMeta pack_step_meta(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                        const std::vector<int32_t>& block_table, size_t ctx_before, size_t seq_after,
                        size_t block_size, int32_t state_in_slot = -1, int32_t state_out_slot = -1,
                        bool has_initial_state = false);

// ---- prefix-shared pages (radix.rs:1-1041, 1129-1157, 1234-1245) -------------------------------
// A radix tree over token ids whose edges are whole pages: a node holds a run of pages (key =
// tokens, value = physical page ids, optionally the draft model's pages beside them) and,
// optionally, the handle of a recurrent-state snapshot taken at the end of its key.  The handle
// is opaque here (the state pools are not part of this library); what the tree does with it is
// what keeps the page side correct: a prefix only counts as a hit up to the deepest node that
// still has a snapshot, internal nodes may lose theirs (tombstones) while their pages stay for
// longer descendants, leaves never are tombstones.
//
// Two lock counts per node: full_lock_ref pins the pages of every node on [node .. root),
// state_lock_ref pins the snapshot of the locked node alone (full >= state everywhere).  Two
// recency orders: a hit refreshes the page order along the whole path and the snapshot order on
// the hit node only.  Both orders are intrusive doubly linked lists through the node arena, so a
// touch is O(1).
struct PrefixMatch {
    size_t kv_matched_tokens = 0;    // whole-page prefix present in the tree, snapshot or not
    size_t matched_tokens = 0;       // usable prefix: up to last_node (multiple of page_size)
    std::vector<int32_t> kv_pages;   // matched_tokens / page_size shared pages, in sequence order
    std::vector<int32_t> draft_pages;
    bool has_state = false;          // false only when nothing matched
    int32_t state_slot = -1;
    int last_node = 0;               // deepest matched node with a snapshot; 0 = root
    size_t state_branching_seqlen = 0;  // > 0: pages matched past last_node; chunk-aligned length
};
struct PrefixInsertResult {
    size_t existing_prefix_tokens = 0;   // tokens of the insert that were in the tree already
    bool state_already_existed = false;  // true: the caller keeps (frees) the handle it offered
    std::vector<int32_t> freed_duplicate_kv_pages;  // caller's pages superseded by tree pages
    std::vector<int32_t> freed_duplicate_draft_pages;
    int terminal_node = 0;
};
struct EvictResult {
    std::vector<int32_t> freed_kv_pages;
    std::vector<int32_t> freed_draft_pages;
    std::vector<int32_t> freed_state_slots;
};

class PrefixPageCache {
public:
    // state_chunk_tokens: spacing of snapshots, a multiple of page_size (0 = page_size).
    explicit PrefixPageCache(size_t page_size, size_t state_chunk_tokens = 0);
    void reset();
    size_t page_size() const { return page_size_; }
    size_t state_chunk_tokens() const { return chunk_; }
    bool disable = false;  // every call becomes a no-op / miss (radix.rs:392,497,563)

    // Longest whole-page prefix of token_ids that ends in a node with a snapshot
    // (radix.rs:383-490).  A partial match of a node splits it.  Refreshes both recency orders.
    PrefixMatch match_prefix(const std::vector<int32_t>& token_ids);
    // radix.rs:494-550.  dec on a count of zero throws std::logic_error.
    void inc_lock_ref(int node);
    void dec_lock_ref(int node);
    // Donates page-aligned (token_ids, kv_pages[, draft_pages], state_slot) (radix.rs:552-699).
    // The first prev_protected_pages pages are the tree's own (the request got them from a hit);
    // pages behind them whose tokens are already cached are returned as duplicates.
    // Throws std::invalid_argument on lengths that do not fit.
    PrefixInsertResult insert(const std::vector<int32_t>& token_ids, const std::vector<int32_t>& kv_pages,
                              const std::vector<int32_t>& draft_pages, int32_t state_slot,
                              size_t prev_protected_pages);
    // Deletes unlocked leaves, least recently used first, decode tails before anything else, until
    // at least num_pages pages are free; tombstone ancestors that become leaves go with them
    // (radix.rs:701-756, 950-981).
    EvictResult evict_full_pages(size_t num_pages);
    // Frees snapshots (radix.rs:907-948): superseded single-child internal nodes first (no page
    // freed), then reclaimable decode-tail leaves, then snapshot recency order.
    EvictResult evict_state_slots(size_t num_slots);
    bool has_evictable_internal_state() const;
    // Drops every node's claim on `slot` (radix.rs:856-886); `slot` itself is not reported back.
    EvictResult invalidate_state_slot(int32_t slot);
    // radix.rs:772-776: the leaf holds generated tokens nobody has verified yet.
    void mark_node_decode_tail(int node);
    bool can_recycle_locked_state(int node) const;  // radix.rs:838-844
    // Takes the snapshot handle of an unlocked-state internal node (radix.rs:888-899); -1 if none.
    int32_t reclaim_internal_state(int node);
    void set_node_state(int node, int32_t slot);  // a live node without a snapshot gets one
    std::vector<int32_t> collect_node_kv_pages(int node) const;  // radix.rs:180-193

    size_t full_evictable_pages() const { return full_evictable_pages_; }
    size_t full_protected_pages() const { return full_protected_pages_; }
    size_t state_evictable_slots() const { return state_evictable_slots_; }
    size_t state_protected_slots() const { return state_protected_slots_; }
    size_t cached_pages() const { return full_evictable_pages_ + full_protected_pages_; }
    bool node_alive(int node) const { return node >= 0 && (size_t)node < nodes_.size() && nodes_[node].alive; }
    size_t arena_size() const { return nodes_.size(); }
    uint64_t total_lookups = 0, total_lookup_tokens = 0, total_hit_tokens = 0, total_state_hits = 0;
    double hit_rate() const { return total_lookup_tokens ? (double)total_hit_tokens / (double)total_lookup_tokens : 0.0; }
    // Recomputes the four counters and checks the lock / tombstone / list invariants
    // (radix.rs:983-1041); on failure returns false and says why.
    bool sanity_check(std::string* why = nullptr) const;

private:
    struct Node {
        int parent = -1;
        std::map<std::vector<int32_t>, int> children;  // keyed by the child's first page
        std::vector<int32_t> key, pages, draft_pages;
        bool has_state = false;
        int32_t state_slot = -1;
        size_t full_lock_ref = 0, state_lock_ref = 0;
        bool decode_tail = false, alive = false;
        int lru_prev[2] = {-1, -1}, lru_next[2] = {-1, -1};  // [0] page order, [1] snapshot order
        bool in_lru[2] = {false, false};
    };
    enum { kFull = 0, kState = 1 };
    int alloc_node();
    void retire(int id);
    void lru_push_mru(int which, int id);
    void lru_remove(int which, int id);
    void lru_touch(int which, int id);
    void touch_path(int node);
    size_t common_pages(const std::vector<int32_t>& key, const int32_t* rest, size_t rest_len) const;
    int split_node(int child, size_t split_tokens);
    void delete_leaf(int leaf, EvictResult* out);
    bool has_verified_state_below(int node) const;
    bool superseded_linear_internal(int node) const;
    bool reclaimable_decode_tail_leaf(int node) const;

    std::vector<Node> nodes_;
    std::vector<int> free_ids_;
    int lru_head_[2] = {-1, -1}, lru_tail_[2] = {-1, -1};  // head = least recently used
    size_t page_size_, chunk_;
    size_t full_evictable_pages_ = 0, full_protected_pages_ = 0;
    size_t state_evictable_slots_ = 0, state_protected_slots_ = 0;
};

// A request's page list: shared prefix pages first (protected), private pages behind them.
struct RequestPages {
    std::vector<int32_t> token_ids;  // committed tokens
    std::vector<int32_t> kv_pages;
    std::vector<int32_t> draft_pages;
    size_t protected_pages = 0;
    int last_locked_node = 0;
    size_t page_size = 0;

    // Binds a prefix hit: clones the shared pages and locks their path (radix.rs:1129-1157).
    void restore_prefix_hit(PrefixPageCache& cache, const std::vector<int32_t>& prompt_tokens,
                            const PrefixMatch& m);
    // Drops private tail pages beyond ceil(committed / page_size); never a protected page
    // (radix.rs:1234-1245).  Returns the pages to hand back to the pool.
    std::vector<int32_t> rollback_uncommitted_kv_pages();
    // The page side of a donation (radix.rs:1247-1380): the first cache_len committed tokens
    // (page-aligned, beyond the protected prefix) and their pages go to the tree with the snapshot
    // handle state_slot; pages the tree already had are swapped for the tree's and the request's
    // copies returned; the lock moves to the new terminal node, or is dropped when the request
    // finishes, in which case the private tail pages are returned as well and a leaf that extends
    // a protected prompt is marked as an unverified decode tail.
    struct Donation {
        size_t donated_seq_len = 0;
        bool state_already_existed = false;
        std::vector<int32_t> freed_kv_pages, freed_draft_pages;
    };
    Donation donate_pages(PrefixPageCache& cache, size_t cache_len, int32_t state_slot, bool finish_req);
};

// Grows dst to target_pages: evicts the deficit from the prefix cache in one batch, then takes
// ascending pages from the pool; returns false (dst unchanged) if that is still not enough
// (batch.rs:57-93).
bool reserve_kv_pages_from(KvPool& pool, PrefixPageCache& cache, std::vector<int32_t>* dst, size_t target_pages);
void free_kv_pages(KvPool& pool, const std::vector<int32_t>& pages);

}  // namespace warp34_host
