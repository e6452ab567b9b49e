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

// ---- prefix-shared pages (radix.rs page side) -------------------------------------------------
struct PrefixMatch {
    size_t matched_tokens = 0;       // whole pages only
    std::vector<int32_t> kv_pages;   // shared physical pages, in sequence order
    int last_node = 0;               // 0 = root (nothing matched)
};
struct EvictResult {
    std::vector<int32_t> freed_kv_pages;
};

// Page-granular prefix tree over token ids: each node owns exactly one full page.  Nodes on a
// locked path are never evicted; eviction removes least-recently-used unlocked leaves.
class PrefixPageCache {
public:
    explicit PrefixPageCache(size_t page_size);
    size_t page_size() const { return page_size_; }
    // Longest whole-page prefix of token_ids already cached (radix.rs:383-490); refreshes LRU.
    PrefixMatch match_prefix(const std::vector<int32_t>& token_ids);
    // Locks / unlocks the path [node .. root) (radix.rs:494-550).
    void inc_lock_ref(int node);
    void dec_lock_ref(int node);
    // Donates the whole pages of (token_ids, kv_pages) to the tree.  Pages whose prefix is
    // already cached under another physical page are returned as duplicates for the caller to
    // free; returns the node of the last whole page.
    int insert(const std::vector<int32_t>& token_ids, const std::vector<int32_t>& kv_pages,
               std::vector<int32_t>* duplicate_pages);
    // Evicts up to num_pages unlocked leaf pages, least recently used first (radix.rs:950-981).
    EvictResult evict_full_pages(size_t num_pages);
    size_t full_evictable_pages() const;
    size_t full_protected_pages() const;
    size_t cached_pages() const { return live_nodes_; }

private:
    struct Node {
        int parent = -1;
        std::vector<int32_t> key;  // page_size tokens
        int32_t page = -1;
        int lock_ref = 0;
        uint64_t last_use = 0;
        std::map<std::vector<int32_t>, int> children;
        bool live = false;
    };
    std::vector<Node> nodes_;
    std::vector<int> free_ids_;
    size_t page_size_;
    size_t live_nodes_ = 0;
    uint64_t clock_ = 0;
};

// A request's page list: shared prefix pages first (protected), private pages behind them.
struct RequestPages {
    std::vector<int32_t> token_ids;  // committed tokens
    std::vector<int32_t> kv_pages;
    size_t protected_pages = 0;
    int last_locked_node = 0;
    size_t page_size = 0;

    // Binds a prefix hit: clones the shared pages and locks their path (radix.rs:1129-1157).
    void restore_prefix_hit(PrefixPageCache& cache, const std::vector<int32_t>& prompt_tokens,
                            const PrefixMatch& m);
    // Drops private tail pages beyond ceil(committed / page_size); never a protected page
    // (radix.rs:1234-1245).  Returns the pages to hand back to the pool.
    std::vector<int32_t> rollback_uncommitted_kv_pages();
};

// Grows dst to target_pages: evicts the deficit from the prefix cache in one batch, then takes
// ascending pages from the pool; returns false (dst unchanged) if that is still not enough
// (batch.rs:57-93).
bool reserve_kv_pages_from(KvPool& pool, PrefixPageCache& cache, std::vector<int32_t>* dst, size_t target_pages);
void free_kv_pages(KvPool& pool, const std::vector<int32_t>& pages);

}  // namespace warp34_host
