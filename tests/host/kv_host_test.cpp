// Host-logic tests; cases follow the reference's own unit tests
// (crates/warp34-host/src/cache.rs:628-826, model/graph_io.rs:1286) plus the page-reservation
// and prefix-sharing behaviour of model/batch.rs:57-93 and radix.rs (its own test module,
// radix.rs:1403-1742, and tests/radix_cache_and_scheduler.rs:16-93).
// Prints one "ok <name>" line per passing test; exits non-zero at the first failure.
#include <cstdio>
#include <cstdlib>
#include <set>
#include <stdexcept>
#include <string>

#include "../../warp34_amd/host/graph_io.h"
#include "../../warp34_amd/host/kv_host.h"

using namespace warp34_host;

#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) {                                                           \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
            std::exit(1);                                                        \
        }                                                                        \
    } while (0)

// host-memory stand-in for the device allocator: the pool logic only needs addresses
struct HostAllocator final : DeviceAllocator {
    std::set<uint64_t> live;
    size_t fail_after = ~size_t(0);
    int alloc(int, size_t bytes, uint64_t* addr) override {
        if (live.size() >= fail_after) return 2;  // hipErrorOutOfMemory
        void* p = std::malloc(bytes ? bytes : 1);
        *addr = (uint64_t)(uintptr_t)p;
        live.insert(*addr);
        return 0;
    }
    void release(int, uint64_t addr) override {
        CHECK(live.erase(addr) == 1);
        std::free((void*)(uintptr_t)addr);
    }
};

static void test_row_bytes() {
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_FP16, 256) == 512);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_BF16, 256) == 512);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_TQ4, 256) == 132);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_Q8_0, 256) == 272);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_FP8_E4M3, 256) == 264);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_FP16, 128) == 256);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_TQ4, 128) == 66);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_Q8_0, 128) == 136);
    CHECK(kv_format_row_bytes(WARP34_KV_FORMAT_FP8_E4M3, 128) == 132);
    std::puts("ok row_bytes");
}

static void test_policy_resolution() {
    const size_t n = 16;
    const int id = WARP34_KV_TRANSFORM_IDENTITY, wht = WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
    for (size_t l = 0; l < n; ++l) {
        CHECK((resolve_layer(KvFormatPolicy::Fp16, l, n) == LayerFormats{WARP34_KV_FORMAT_FP16, WARP34_KV_FORMAT_FP16, id, id}));
        CHECK((resolve_layer(KvFormatPolicy::Bf16, l, n) == LayerFormats{WARP34_KV_FORMAT_BF16, WARP34_KV_FORMAT_BF16, id, id}));
        CHECK((resolve_layer(KvFormatPolicy::Tq4All, l, n) == LayerFormats{WARP34_KV_FORMAT_TQ4, WARP34_KV_FORMAT_TQ4, wht, wht}));
        CHECK((resolve_layer(KvFormatPolicy::Fp8, l, n) ==
               LayerFormats{WARP34_KV_FORMAT_FP8_E4M3, WARP34_KV_FORMAT_FP8_E4M3, id, id}));
        const bool anchor = l >= n - 4;
        const LayerFormats plain = resolve_layer(KvFormatPolicy::Tq4, l, n);
        const LayerFormats fp8 = resolve_layer_with_fp8(KvFormatPolicy::Tq4, l, n, true);
        if (anchor) {
            CHECK((plain == LayerFormats{WARP34_KV_FORMAT_Q8_0, WARP34_KV_FORMAT_Q8_0, id, id}));
            CHECK((fp8 == LayerFormats{WARP34_KV_FORMAT_FP8_E4M3, WARP34_KV_FORMAT_FP8_E4M3, id, id}));
        } else {
            CHECK((plain == LayerFormats{WARP34_KV_FORMAT_TQ4, WARP34_KV_FORMAT_TQ4, wht, wht}));
            CHECK((fp8 == plain));
        }
    }
    // fewer than four layers: every layer is an anchor (saturating subtraction)
    CHECK(resolve_layer(KvFormatPolicy::Tq4, 0, 3).k_format == WARP34_KV_FORMAT_Q8_0);
    std::puts("ok policy_resolution");
}

static void test_bytes_per_token() {
    CHECK(bytes_per_token(KvFormatPolicy::Fp16, 16, 8, 256) == 16 * 8 * (512 + 512));
    CHECK(bytes_per_token(KvFormatPolicy::Tq4All, 16, 8, 256) == 16 * 8 * (132 + 132));
    CHECK(bytes_per_token(KvFormatPolicy::Tq4, 16, 8, 256) == 4 * 8 * 544 + 12 * 8 * 264);
    CHECK(bytes_per_token(KvFormatPolicy::Fp8, 16, 8, 256) == 16 * 8 * (264 + 264));
    CHECK(bytes_per_token_with_fp8(KvFormatPolicy::Tq4, 16, 8, 256, true) == 4 * 8 * 528 + 12 * 8 * 264);
    // 27B figures: 16 layers x 4 kv heads (tests/tq4_vision_and_moe.rs:51-54)
    CHECK(bytes_per_token(KvFormatPolicy::Fp16, 16, 4, 256) == 65536);
    CHECK(bytes_per_token(KvFormatPolicy::Q8_0, 16, 4, 256) == 34816);
    CHECK(bytes_per_token(KvFormatPolicy::Tq4, 16, 4, 256) == 21376);
    CHECK(bytes_per_token(KvFormatPolicy::Tq4All, 16, 4, 256) == 16896);
    std::puts("ok bytes_per_token");
}

static void test_policy_names() {
    for (const char* s : {"fp16", "bf16", "q8_0", "fp8", "tq4", "tq4_all"}) {
        const auto p = parse_kv_policy(s);
        CHECK(p.has_value());
        CHECK(std::string(kv_policy_name(*p)) == s);
    }
    CHECK(!parse_kv_policy("int4").has_value());
    std::puts("ok policy_names");
}

static void test_page_bitmap() {
    PageBitmap bm(130);
    CHECK(bm.free_count() == 130);
    for (int expected = 0; expected < 130; ++expected) CHECK(bm.alloc() == std::optional<int32_t>(expected));
    CHECK(!bm.alloc().has_value());
    CHECK(bm.free_count() == 0);
    for (int p : {129, 64, 65, 3, 2, 1, 0, 128, 63}) bm.free(p);
    bm.free(64);   // duplicate
    bm.free(-1);   // out of range
    bm.free(130);  // out of range
    CHECK(bm.free_count() == 9);
    const int want[9] = {0, 1, 2, 3, 63, 64, 65, 128, 129};
    for (int i = 0; i < 9; ++i) CHECK(bm.alloc() == std::optional<int32_t>(want[i]));
    CHECK(!bm.alloc().has_value());
    bm.reset();
    CHECK(bm.free_count() == 130);
    CHECK(bm.alloc() == std::optional<int32_t>(0));
    // a free below the cursor pulls the cursor back; one above it is found after wrap-around
    PageBitmap b2(256);
    for (int i = 0; i < 200; ++i) b2.alloc();
    b2.free(10);
    CHECK(b2.alloc() == std::optional<int32_t>(10));
    CHECK(b2.alloc() == std::optional<int32_t>(200));
    std::puts("ok page_bitmap");
}

static void test_kv_pool_layout() {
    HostAllocator ha;
    {
        KvPool pool;
        const std::vector<size_t> layer_ids = {3, 7, 11, 15, 19, 23};
        HostError e = KvPool::new_target_full_attn(&pool, ha, 0, layer_ids, 2, 256, 64, 40, KvFormatPolicy::Tq4, false);
        CHECK(!e);
        CHECK(pool.layers.size() == 6 && ha.live.size() == 12);
        // TQ4 layers: token 132, head 64*132, page 2*64*132 (same strides for K and V)
        const warp34_kv_layer_layout& L0 = pool.layers[0].layout;
        CHECK(L0.k_token_stride_bytes == 132 && L0.k_head_stride_bytes == 8448 && L0.k_page_stride_bytes == 16896);
        CHECK(L0.v_token_stride_bytes == 132 && L0.v_head_stride_bytes == 8448 && L0.v_page_stride_bytes == 16896);
        CHECK(L0.k_format == WARP34_KV_FORMAT_TQ4 && L0.k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256);
        CHECK(L0.layer_id == 3 && L0.namespace_id == WARP34_KV_NAMESPACE_TARGET_FULL_ATTN);
        CHECK(L0.local_kv_heads == 2 && L0.head_dim == 256 && L0.block_size == 64 && L0.reserved == 0);
        CHECK(pool.layers[0].k_bytes == 40u * 16896u);
        // last four layers are the Q8_0 anchors
        const warp34_kv_layer_layout& L5 = pool.layers[5].layout;
        CHECK(L5.k_format == WARP34_KV_FORMAT_Q8_0 && L5.k_token_stride_bytes == 272 && L5.layer_id == 23);
        CHECK(pool.layers[1].layout.k_format == WARP34_KV_FORMAT_TQ4);
        CHECK(pool.layers[2].layout.k_format == WARP34_KV_FORMAT_Q8_0);
        // pages
        CHECK(pool.free_count() == 40);
        CHECK(pool.alloc_page() == std::optional<int32_t>(0));
        pool.truncate_pages(100);  // never grows
        CHECK(pool.num_pages == 40 && pool.free_count() == 39);
        pool.truncate_pages(8);
        CHECK(pool.num_pages == 8 && pool.free_count() == 8);
        // bf16 pool: 512-byte rows
        KvPool bf;
        CHECK(!KvPool::new_target_full_attn(&bf, ha, 0, {0}, 2, 256, 64, 4, KvFormatPolicy::Bf16, false));
        CHECK(bf.layers[0].layout.k_head_stride_bytes == 32768 && bf.layers[0].layout.k_page_stride_bytes == 65536);
        // fp8 policy without hardware support
        KvPool bad;
        HostError e2 = KvPool::new_target_full_attn(&bad, ha, 0, {0}, 2, 256, 64, 4, KvFormatPolicy::Fp8, false);
        CHECK(e2.code == -23);
        // allocation failure surfaces the allocator's code and leaks nothing
        ha.fail_after = ha.live.size() + 1;
        KvPool oom;
        HostError e3 = KvPool::new_target_full_attn(&oom, ha, 0, {0, 1}, 2, 256, 64, 4, KvFormatPolicy::Tq4All, false);
        CHECK(e3.code == 2);
        ha.fail_after = ~size_t(0);
    }
    CHECK(ha.live.empty());
    std::puts("ok kv_pool_layout");
}

static void test_slot_mapping_and_step_blob() {
    // model/graph_io.rs:1286: block table [7, 3], page 16, positions 15 and 16
    const std::vector<int32_t> bt = {7, 3};
    const std::vector<int32_t> s = write_slot_mapping(bt, 15, 17, 16);
    CHECK(s.size() == 2 && s[0] == 7 * 16 + 15 && s[1] == 3 * 16);
    CHECK(write_slot_mapping(bt, 5, 5, 16).empty());
    const StepMeta m = pack_step_meta({101, 102}, {15, 16}, bt, 15, 17, 16, 4, 5, true);
    const std::vector<int32_t> want = {101, 102, 15, 16, 7 * 16 + 15, 48, 7, 3, 0, 2, 15, 17, 4, 5, 1};
    CHECK(m.words == want);
    const uint64_t base = 0x10000;
    const warp34_attention_batch b = m.batch_at(base, WARP34_ATTN_MASK_CAUSAL, 0.0625f);
    CHECK((uint64_t)(uintptr_t)b.write_slot_mapping == base + 16);
    CHECK((uint64_t)(uintptr_t)b.block_tables == base + 24);
    CHECK((uint64_t)(uintptr_t)b.query_start_loc == base + 32);
    CHECK((uint64_t)(uintptr_t)b.context_lens_before == base + 40);
    CHECK((uint64_t)(uintptr_t)b.seq_lens_after == base + 44);
    CHECK(b.num_reqs == 1 && b.total_tokens == 2 && b.max_blocks_per_req == 2 && b.max_q_len == 2 && b.max_seq_len == 17);
    CHECK(b.valid_token_mask == nullptr && b.valid_req_mask == nullptr && b.sm_scale == 0.0625f);
    CHECK(m.positions_at(base) == base + 8);
    std::puts("ok slot_mapping_and_step_blob");
}

static std::vector<int32_t> iota_tokens(int n, int salt) {
    std::vector<int32_t> t(n);
    for (int i = 0; i < n; ++i) t[i] = salt * 100000 + i;
    return t;
}

static std::vector<int32_t> range(int lo, int hi) {
    std::vector<int32_t> t;
    for (int i = lo; i < hi; ++i) t.push_back(i);
    return t;
}
static std::vector<int32_t> cat(std::vector<int32_t> a, const std::vector<int32_t>& b) {
    a.insert(a.end(), b.begin(), b.end());
    return a;
}
using Pages = std::vector<int32_t>;
#define SANE(cache)                                                              \
    do {                                                                         \
        std::string why_;                                                        \
        if (!(cache).sanity_check(&why_)) {                                      \
            std::printf("FAILED %s:%d: sanity_check: %s\n", __FILE__, __LINE__, why_.c_str()); \
            std::exit(1);                                                        \
        }                                                                        \
    } while (0)

static void test_reservation_and_prefix_sharing() {
    HostAllocator ha;
    KvPool pool;
    CHECK(!KvPool::new_target_full_attn(&pool, ha, 0, {0}, 2, 256, 16, 12, KvFormatPolicy::Tq4All, false));
    PrefixPageCache cache(16, 16);

    // request A: 70 tokens -> 5 pages, ascending page ids
    RequestPages a;
    a.page_size = 16;
    CHECK(reserve_kv_pages_from(pool, cache, &a.kv_pages, 5));
    CHECK((a.kv_pages == Pages{0, 1, 2, 3, 4}));
    CHECK(reserve_kv_pages_from(pool, cache, &a.kv_pages, 3));  // already satisfied
    a.token_ids = iota_tokens(70, 1);
    // A finishes: its four whole pages are donated, the partial fifth goes back to the pool
    const RequestPages::Donation da = a.donate_pages(cache, 64, 500, true);
    CHECK(da.donated_seq_len == 64 && (da.freed_kv_pages == Pages{4}) && cache.cached_pages() == 4);
    free_kv_pages(pool, da.freed_kv_pages);
    CHECK(pool.free_count() == 8 && cache.full_evictable_pages() == 4);
    SANE(cache);

    // request B shares the first 40 tokens of A: the tree holds two of its whole pages, but the
    // only snapshot sits at 64 tokens, so nothing is usable yet (the node is cut at 32 tokens)
    std::vector<int32_t> prompt_b = iota_tokens(40, 1);
    for (int i = 0; i < 30; ++i) prompt_b.push_back(900000 + i);
    const PrefixMatch miss = cache.match_prefix(prompt_b);
    CHECK(miss.kv_matched_tokens == 32 && miss.matched_tokens == 0 && !miss.has_state && miss.last_node == 0);
    CHECK(miss.state_branching_seqlen == 32);
    // a snapshot at 32 tokens (another request's checkpoint) turns the cut into a hit
    const PrefixInsertResult mid = cache.insert(iota_tokens(32, 1), {0, 1}, {}, 501, 2);
    CHECK(!mid.state_already_existed && mid.existing_prefix_tokens == 32 && mid.freed_duplicate_kv_pages.empty());
    const PrefixMatch mb = cache.match_prefix(prompt_b);
    CHECK(mb.matched_tokens == 32 && (mb.kv_pages == Pages{0, 1}) && mb.has_state && mb.state_slot == 501);
    RequestPages b;
    b.restore_prefix_hit(cache, prompt_b, mb);
    CHECK(b.protected_pages == 2 && b.token_ids.size() == 32 && cache.full_protected_pages() == 2);
    SANE(cache);
    // B needs ceil(70/16) = 5 pages: three private ones, lowest free ids first
    CHECK(reserve_kv_pages_from(pool, cache, &b.kv_pages, 5));
    CHECK((b.kv_pages == Pages{0, 1, 4, 5, 6}));

    // speculative tail: B reserves two more pages, commits only up to 85 tokens, rolls back
    b.token_ids = prompt_b;
    CHECK(reserve_kv_pages_from(pool, cache, &b.kv_pages, 7));
    b.token_ids.resize(70);
    for (int i = 0; i < 15; ++i) b.token_ids.push_back(i);
    const Pages rolled = b.rollback_uncommitted_kv_pages();
    CHECK((rolled == Pages{8}) && b.kv_pages.size() == 5 + 1);
    free_kv_pages(pool, rolled);
    // rollback never drops a shared page even when nothing is committed
    RequestPages c = b;
    c.token_ids.clear();
    const Pages rolled_c = c.rollback_uncommitted_kv_pages();
    CHECK(c.kv_pages.size() == 2 && rolled_c.size() == 4);

    // pool pressure: 12 pages, cache holds 0..3 (0 and 1 locked), B holds 4,5,6,7 -> free 8..11
    CHECK(pool.free_count() == 4);
    Pages big;
    CHECK(reserve_kv_pages_from(pool, cache, &big, 6));  // evicts the two unlocked cached pages
    CHECK(cache.cached_pages() == 2 && cache.full_evictable_pages() == 0);
    CHECK((big == Pages{2, 3, 8, 9, 10, 11}));
    Pages more;
    CHECK(!reserve_kv_pages_from(pool, cache, &more, 1));  // locked pages cannot be evicted
    CHECK(more.empty());
    cache.dec_lock_ref(b.last_locked_node);
    CHECK(reserve_kv_pages_from(pool, cache, &more, 2));
    CHECK((more == Pages{0, 1}) && cache.cached_pages() == 0);
    SANE(cache);

    // duplicate donation: same tokens under other physical pages are handed back
    PrefixPageCache c2(16);
    const std::vector<int32_t> t = iota_tokens(32, 7);
    c2.insert(t, {20, 21}, {}, 1, 0);
    const PrefixInsertResult d2 = c2.insert(t, {30, 31}, {}, 2, 0);
    CHECK((d2.freed_duplicate_kv_pages == Pages{30, 31}) && d2.state_already_existed && c2.cached_pages() == 2);
    std::puts("ok reservation_and_prefix_sharing");
}

// ---- the reference's own cases for the tree (radix.rs:1403-1742, tests/radix_cache_and_scheduler.rs:16-93),
// ---- the snapshot handles being plain numbers here ----
static void test_radix_initialization() {  // radix.rs:1403-1411
    PrefixPageCache cache(16, 64);
    CHECK(cache.page_size() == 16 && cache.state_chunk_tokens() == 64);
    CHECK(cache.total_lookups == 0 && cache.total_hit_tokens == 0);
    SANE(cache);
    bool threw = false;
    try {
        PrefixPageCache bad(16, 40);
    } catch (const std::invalid_argument&) {
        threw = true;
    }
    CHECK(threw);
    std::puts("ok radix_initialization");
}

static void test_radix_insert_exact_and_match() {  // radix.rs:1413-1451
    PrefixPageCache cache(16, 64);
    const auto tokens = range(0, 64);
    const Pages kv{101, 102, 103, 104}, draft{201, 202, 203, 204};
    const PrefixInsertResult ins = cache.insert(tokens, kv, draft, 42, 0);
    CHECK(ins.existing_prefix_tokens == 0 && !ins.state_already_existed && ins.freed_duplicate_kv_pages.empty());
    SANE(cache);
    const PrefixMatch m = cache.match_prefix(tokens);
    CHECK(m.matched_tokens == 64 && m.kv_pages == kv && m.draft_pages == draft);
    CHECK(m.has_state && m.state_slot == 42 && m.last_node == ins.terminal_node);
    const PrefixMatch longer = cache.match_prefix(cat(tokens, {999, 1000}));
    CHECK(longer.matched_tokens == 64 && longer.state_slot == 42);
    // 48 tokens cut the node into a 48-token part without a snapshot and a 16-token leaf: the
    // pages are there, nothing is usable
    const PrefixMatch shorter = cache.match_prefix(range(0, 48));
    CHECK(shorter.kv_matched_tokens == 48 && shorter.matched_tokens == 0 && !shorter.has_state);
    SANE(cache);
    CHECK(cache.total_lookups == 3 && cache.total_lookup_tokens == 64 + 66 + 48 && cache.total_hit_tokens == 128);
    std::puts("ok radix_insert_exact_and_match");
}

static void test_radix_split_and_branch() {  // radix.rs:1453-1487
    PrefixPageCache cache(16, 64);
    const auto tokens_a = range(0, 64);
    cache.insert(tokens_a, {1, 2, 3, 4}, {}, 10, 0);
    SANE(cache);
    const auto tokens_b = cat(range(0, 32), range(100, 132));
    const PrefixInsertResult ins_b = cache.insert(tokens_b, {1, 2, 5, 6}, {}, 20, 0);
    CHECK(ins_b.existing_prefix_tokens == 32 && (ins_b.freed_duplicate_kv_pages == Pages{1, 2}));
    SANE(cache);
    const PrefixMatch ma = cache.match_prefix(tokens_a);
    CHECK(ma.matched_tokens == 64 && ma.state_slot == 10 && (ma.kv_pages == Pages{1, 2, 3, 4}));
    const PrefixMatch mb = cache.match_prefix(tokens_b);
    CHECK(mb.matched_tokens == 64 && mb.state_slot == 20 && (mb.kv_pages == Pages{1, 2, 5, 6}));
    std::puts("ok radix_split_and_branch");
}

static void test_radix_dual_lock_and_eviction() {  // radix.rs:1489-1516
    PrefixPageCache cache(16, 64);
    const PrefixInsertResult ins = cache.insert(range(0, 64), {10, 20, 30, 40}, {}, 99, 0);
    cache.inc_lock_ref(ins.terminal_node);
    SANE(cache);
    CHECK(cache.evict_full_pages(4).freed_kv_pages.empty());
    CHECK(cache.evict_state_slots(1).freed_state_slots.empty());
    cache.dec_lock_ref(ins.terminal_node);
    SANE(cache);
    bool threw = false;
    try {
        cache.dec_lock_ref(ins.terminal_node);
    } catch (const std::logic_error&) {
        threw = true;
    }
    CHECK(threw);
    const EvictResult ev = cache.evict_full_pages(4);
    CHECK((ev.freed_kv_pages == Pages{10, 20, 30, 40}) && (ev.freed_state_slots == Pages{99}));
    SANE(cache);
    std::puts("ok radix_dual_lock_and_eviction");
}

static void test_radix_rollback_and_lru_order() {  // radix.rs:1548-1594, parts 2 and 3
    RequestPages req;
    req.page_size = 16;
    req.kv_pages = range(100, 116);  // room for 256 tokens, 200 committed
    req.protected_pages = 4;
    req.token_ids = range(0, 200);
    const Pages freed = req.rollback_uncommitted_kv_pages();
    CHECK((freed == Pages{113, 114, 115}) && req.kv_pages.size() == 13);

    PrefixPageCache cache(16, 64);
    const auto a = range(0, 64), b = range(100, 164), c = range(200, 264);
    cache.insert(a, {1, 2, 3, 4}, {}, 11, 0);
    cache.insert(b, {5, 6, 7, 8}, {}, 22, 0);
    cache.insert(c, {9, 10, 11, 12}, {}, 33, 0);
    CHECK(cache.match_prefix(a).state_slot == 11);  // order is now b, c, a
    CHECK(cache.state_evictable_slots() == 3);
    CHECK((cache.evict_state_slots(1).freed_state_slots == Pages{22}));
    CHECK((cache.evict_state_slots(1).freed_state_slots == Pages{33}));
    CHECK((cache.evict_state_slots(1).freed_state_slots == Pages{11}));
    CHECK(cache.state_evictable_slots() == 0 && cache.cached_pages() == 0);
    SANE(cache);
    std::puts("ok radix_rollback_and_lru_order");
}

static void test_radix_superseded_linear_turns() {  // radix.rs:1596-1621
    PrefixPageCache cache(16, 64);
    const auto s0 = range(0, 64);
    cache.insert(s0, {1, 2, 3, 4}, {}, 10, 0);
    const auto s1 = range(1000, 1128);
    cache.insert(range(1000, 1064), {10, 11, 12, 13}, {}, 20, 0);
    cache.insert(s1, {10, 11, 12, 13, 14, 15, 16, 17}, {}, 21, 4);
    CHECK(cache.has_evictable_internal_state());
    // under pressure the overtaken checkpoint of session 1 goes (no page freed), not the waiting
    // leaf of session 0
    const EvictResult ev = cache.evict_state_slots(1);
    CHECK((ev.freed_state_slots == Pages{20}) && ev.freed_kv_pages.empty());
    const PrefixMatch hit = cache.match_prefix(s0);
    CHECK(hit.matched_tokens == 64 && hit.state_slot == 10);
    SANE(cache);
    std::puts("ok radix_superseded_linear_turns");
}

static void test_radix_decode_tail_leaf() {  // radix.rs:1623-1660, the page side of the two donations
    PrefixPageCache cache(16, 64);
    RequestPages req;
    req.page_size = 16;
    const auto prompt = range(0, 64);
    req.kv_pages = {10, 11, 12, 13};
    req.token_ids = prompt;
    const RequestPages::Donation d1 = req.donate_pages(cache, 64, 2, false);
    CHECK(d1.donated_seq_len == 64 && d1.freed_kv_pages.empty() && req.protected_pages == 4);
    CHECK(req.last_locked_node != 0 && cache.full_protected_pages() == 4);
    req.kv_pages.insert(req.kv_pages.end(), {14, 15, 16, 17});
    req.token_ids = cat(prompt, range(1000, 1064));
    const RequestPages::Donation d2 = req.donate_pages(cache, 128, 3, true);
    CHECK(d2.donated_seq_len == 128 && d2.freed_kv_pages.empty() && req.last_locked_node == 0);
    CHECK(cache.full_protected_pages() == 0 && cache.full_evictable_pages() == 8);
    // one snapshot must go: the unverified generated tail, not the prompt's
    const EvictResult ev = cache.evict_state_slots(1);
    CHECK((ev.freed_state_slots == Pages{3}) && (ev.freed_kv_pages == Pages{14, 15, 16, 17}));
    const PrefixMatch hit = cache.match_prefix(cat(prompt, range(2000, 2064)));
    CHECK(hit.matched_tokens == 64 && hit.state_slot == 2);
    SANE(cache);
    // evict_full_pages takes decode tails first, whatever their age
    PrefixPageCache c2(16, 64);
    RequestPages r2;
    r2.page_size = 16;
    r2.kv_pages = {1, 2, 3, 4};
    r2.token_ids = range(0, 64);
    r2.donate_pages(c2, 64, 7, false);
    r2.kv_pages.insert(r2.kv_pages.end(), {5, 6, 7, 8});
    r2.token_ids = range(0, 128);
    r2.donate_pages(c2, 128, 8, true);               // decode tail, oldest insert of the two leaves
    c2.insert(range(500, 564), {20, 21, 22, 23}, {}, 9, 0);
    c2.match_prefix(range(0, 64));                   // prompt refreshed; the tail leaf stays older than 500..
    const EvictResult e2 = c2.evict_full_pages(1);
    CHECK((e2.freed_kv_pages == Pages{5, 6, 7, 8}) && (e2.freed_state_slots == Pages{8}));
    SANE(c2);
    std::puts("ok radix_decode_tail_leaf");
}

static void test_radix_arena_reuse() {  // radix.rs:1662-1686
    PrefixPageCache cache(16, 64);
    for (int session = 0; session < 512; ++session) {
        RequestPages req;
        req.page_size = 16;
        req.token_ids = range(session * 1000, session * 1000 + 128);
        req.kv_pages = range(session * 16, session * 16 + 8);
        const RequestPages::Donation don = req.donate_pages(cache, 128, 4, true);
        CHECK(don.donated_seq_len == 128 && don.freed_kv_pages.empty());
        const EvictResult ev = cache.evict_full_pages(8);
        CHECK(ev.freed_kv_pages.size() == 8 && ev.freed_state_slots.size() == 1);
        SANE(cache);
    }
    CHECK(cache.arena_size() <= 8);
    std::puts("ok radix_arena_reuse");
}

static void test_radix_recycle_and_invalidate() {  // radix.rs:1688-1741, page side
    PrefixPageCache cache(16, 64);
    const auto turn0 = range(0, 64);
    cache.insert(turn0, {1, 2, 3, 4}, {}, 10, 0);
    const auto turn1 = cat(turn0, range(100, 164));
    const PrefixMatch hit = cache.match_prefix(turn1);
    CHECK(hit.matched_tokens == 64 && hit.state_slot == 10);
    RequestPages req;
    req.restore_prefix_hit(cache, turn1, hit);
    CHECK(cache.can_recycle_locked_state(req.last_locked_node));
    const int prev_locked = req.last_locked_node;
    req.kv_pages.insert(req.kv_pages.end(), {5, 6, 7, 8});
    req.token_ids = turn1;
    const RequestPages::Donation don = req.donate_pages(cache, 128, 2, true);
    CHECK(don.donated_seq_len == 128 && don.freed_kv_pages.empty());
    // with no spare handle the finished request moves the old node's handle to the new end
    const int32_t recycled = cache.reclaim_internal_state(prev_locked);
    CHECK(recycled == 10);
    const PrefixMatch end = cache.match_prefix(turn1);
    CHECK(end.matched_tokens == 128 && end.state_slot == 2);
    cache.set_node_state(end.last_node, recycled);
    SANE(cache);
    const PrefixMatch hit1 = cache.match_prefix(turn1);
    CHECK(hit1.matched_tokens == 128 && hit1.state_slot == 10);
    // the handle turns out unusable: the leaf and the tombstone above it go, leaf pages first
    const EvictResult inv = cache.invalidate_state_slot(10);
    CHECK((inv.freed_kv_pages == Pages{5, 6, 7, 8, 1, 2, 3, 4}) && inv.freed_state_slots.empty());
    CHECK(cache.match_prefix(turn1).matched_tokens == 0);
    SANE(cache);
    std::puts("ok radix_recycle_and_invalidate");
}

static void test_radix_dual_lock_dual_lru_tombstone_and_split() {  // tests/radix_cache_and_scheduler.rs:16-83
    PrefixPageCache cache(16, 64);
    const auto tok_a = range(1000, 1128);
    const PrefixInsertResult ins_a = cache.insert(tok_a, range(0, 8), {}, 10, 0);
    CHECK(!ins_a.state_already_existed && cache.full_evictable_pages() == 8 && cache.state_evictable_slots() == 1);
    SANE(cache);
    const auto tok_b = cat(range(1000, 1064), range(2000, 2064));
    const PrefixInsertResult ins_b = cache.insert(tok_b, {0, 1, 2, 3, 8, 9, 10, 11}, {}, 11, 4);
    CHECK(ins_b.existing_prefix_tokens == 64 && !ins_b.state_already_existed && ins_b.freed_duplicate_kv_pages.empty());
    CHECK(cache.full_evictable_pages() == 12 && cache.state_evictable_slots() == 2);
    SANE(cache);
    // the 64-token node the split made has no snapshot; this insert gives it one
    const PrefixInsertResult ins_mid = cache.insert(range(1000, 1064), range(0, 4), {}, 12, 4);
    CHECK(!ins_mid.state_already_existed && cache.state_evictable_slots() == 3);
    SANE(cache);
    // locking leaf B pins its snapshot and the pages of leaf B and of the 64-token node
    cache.inc_lock_ref(ins_b.terminal_node);
    CHECK(cache.full_protected_pages() == 8 && cache.full_evictable_pages() == 4);
    CHECK(cache.state_protected_slots() == 1);
    SANE(cache);
    const PrefixMatch m_a = cache.match_prefix(tok_a);
    CHECK(m_a.matched_tokens == 128 && m_a.state_slot == 10);
    // the least recent unlocked snapshot is the 64-token node's: it becomes a tombstone, its pages stay
    const EvictResult ev1 = cache.evict_state_slots(1);
    CHECK((ev1.freed_state_slots == Pages{12}) && ev1.freed_kv_pages.empty());
    SANE(cache);
    cache.dec_lock_ref(ins_b.terminal_node);
    CHECK(cache.node_alive(0));
    const EvictResult ev_all = cache.evict_full_pages(12);
    CHECK(ev_all.freed_kv_pages.size() == 12 && ev_all.freed_state_slots.size() == 2);
    CHECK(cache.full_evictable_pages() == 0 && cache.state_evictable_slots() == 0);
    SANE(cache);
    std::puts("ok radix_dual_lock_dual_lru_tombstone_and_split");
}

// Random operations against a brute-force model of what must hold whatever the history: pages
// are neither lost nor handed out twice, a hit returns exactly the pages inserted for those
// tokens, counters match a recount.
static void test_radix_random_walk() {
    PrefixPageCache cache(4, 8);
    std::set<int32_t> in_tree;  // pages the tree owns
    int32_t next_page = 0, next_slot = 1000;
    uint64_t rng = 12345;
    auto rnd = [&](int n) {
        rng = rng * 6364136223846793005ull + 1442695040888963407ull;
        return (int)((rng >> 33) % (uint64_t)n);
    };
    std::vector<int> locked;
    for (int step = 0; step < 4000; ++step) {
        const int op = rnd(10);
        // sequences over a tiny alphabet of pages so that prefixes collide often
        std::vector<int32_t> toks;
        const int n_pages = 1 + rnd(5);
        for (int p = 0; p < n_pages; ++p) {
            const int sym = rnd(3);
            for (int i = 0; i < 4; ++i) toks.push_back(sym * 10 + i);
        }
        if (op < 4) {
            Pages pages;
            for (int p = 0; p < n_pages; ++p) pages.push_back(next_page++);
            const PrefixInsertResult r = cache.insert(toks, pages, {}, next_slot++, 0);
            const size_t existing_pages = r.existing_prefix_tokens / 4;
            CHECK(r.freed_duplicate_kv_pages.size() == existing_pages);
            for (size_t p = existing_pages; p < pages.size(); ++p) CHECK(in_tree.insert(pages[p]).second);
            CHECK(cache.collect_node_kv_pages(r.terminal_node).size() == (size_t)n_pages);
        } else if (op < 7) {
            const PrefixMatch m = cache.match_prefix(toks);
            CHECK(m.matched_tokens % 4 == 0 && m.kv_pages.size() == m.matched_tokens / 4 && m.matched_tokens <= m.kv_matched_tokens);
            for (int32_t p : m.kv_pages) CHECK(in_tree.count(p) == 1);
            CHECK((m.last_node == 0) == (m.matched_tokens == 0));
            if (m.last_node != 0) CHECK(cache.collect_node_kv_pages(m.last_node) == m.kv_pages);
            if (m.last_node != 0 && rnd(2) == 0) {
                cache.inc_lock_ref(m.last_node);
                locked.push_back(m.last_node);
            }
        } else if (op == 7 && !locked.empty()) {
            const int i = rnd((int)locked.size());
            cache.dec_lock_ref(locked[i]);
            locked.erase(locked.begin() + i);
        } else if (op == 8) {
            const EvictResult ev = cache.evict_full_pages(1 + rnd(6));
            for (int32_t p : ev.freed_kv_pages) CHECK(in_tree.erase(p) == 1);
        } else {
            const EvictResult ev = cache.evict_state_slots(1 + rnd(2));
            for (int32_t p : ev.freed_kv_pages) CHECK(in_tree.erase(p) == 1);
        }
        SANE(cache);
        CHECK(cache.cached_pages() == in_tree.size());
        for (int node : locked) CHECK(cache.node_alive(node));
    }
    for (int node : locked) cache.dec_lock_ref(node);
    const EvictResult rest = cache.evict_full_pages(1u << 30);
    for (int32_t p : rest.freed_kv_pages) CHECK(in_tree.erase(p) == 1);
    CHECK(in_tree.empty() && cache.cached_pages() == 0 && cache.state_evictable_slots() == 0);
    SANE(cache);
    std::puts("ok radix_random_walk");
}

// ---- step descriptors of captured steps (model/graph_io.rs) ----
static StepSlice spec_slice(std::vector<int32_t> tokens) {  // the fixture of graph_io.rs:1262-1274
    StepSlice s;
    s.tokens = std::move(tokens);
    s.ctx_len_before = 15;
    s.block_table = {7, 3};
    s.state_in_slot = 2;
    s.state_out_slot = 5;
    s.has_initial_state = true;
    s.spec_slots = {8, 9};
    s.checkpoints = {{1, 6}};
    return s;
}

static void test_spec_verify_meta() {  // graph_io.rs:1276-1317
    using M = SpecVerifyMeta;
    const size_t n = M::T, cp = M::CP;
    M m;
    CHECK(pack_spec_verify_meta(spec_slice({41, 42}), kBaseModelLoraId, 16, &m));
    const auto& w = m.words;
    CHECK(w[0] == 41 && w[1] == 42);
    CHECK(w[n] == 15 && w[n + 1] == 16);
    CHECK(w[2 * n] == 7 * 16 + 15 && w[2 * n + 1] == 3 * 16);  // the second token crosses into the next page
    CHECK(w[3 * n] == 8 && w[3 * n + 1] == 9);
    CHECK(w[4 * n] == 6 && w[4 * n + cp] == 1);
    const int32_t q[6] = {0, 2, 15, 17, 2, 5};
    for (int i = 0; i < 6; ++i) CHECK(w[4 * n + 2 * cp + i] == q[i]);
    for (size_t i = 0; i < n; ++i) CHECK(w[4 * n + 2 * cp + 6 + i] == -1);
    M ml;
    CHECK(pack_spec_verify_meta(spec_slice({41, 42}), 3, 16, &ml));
    CHECK(ml.words[4 * n + 2 * cp + 6] == 3 && ml.words[4 * n + 2 * cp + 7] == 3);
    for (size_t i = 2; i < n; ++i) CHECK(ml.words[4 * n + 2 * cp + 6 + i] == kBaseModelLoraId);
    for (size_t base : {size_t(0), n, 2 * n, 3 * n})
        for (size_t i = 2; i < n; ++i) CHECK(w[base + i] == -1);
    for (size_t i = 1; i < cp; ++i) CHECK(w[4 * n + i] == -1);
    // capacity and table checks
    CHECK(!pack_spec_verify_meta(spec_slice(std::vector<int32_t>(n + 1, 1)), -1, 16, &m));
    CHECK(!pack_spec_verify_meta(spec_slice({}), -1, 16, &m));
    StepSlice s = spec_slice({1, 2});
    s.block_table = {7};
    CHECK(!pack_spec_verify_meta(s, -1, 16, &m));
    s.ctx_len_before = ~size_t(0);
    CHECK(!pack_spec_verify_meta(s, -1, 16, &m));
    // other page sizes: position 15 + 1 stays inside a 64-token page
    s = spec_slice({5, 6});
    CHECK(pack_spec_verify_meta(s, -1, 64, &m) && m.words[2 * n] == 7 * 64 + 15 && m.words[2 * n + 1] == 7 * 64 + 16);
    const warp34_attention_batch b = M::batch_at(0x1000, 0x2000, 2, 8, 4096, 0, 0.0625f);
    CHECK((uint64_t)(uintptr_t)b.query_start_loc == 0x1000 + 4 * M::kQStartLoc && b.total_tokens == 2 && b.num_reqs == 1);
    CHECK((uint64_t)(uintptr_t)b.write_slot_mapping == 0x1000 + 4 * 2 * n && b.max_q_len == 2 && b.max_seq_len == 4096);
    std::puts("ok spec_verify_meta");
}

static void test_batched_decode_meta() {  // graph_io.rs:585-595, 789-871
    CHECK(!decode_graph_bucket(0) && *decode_graph_bucket(1) == 1 && *decode_graph_bucket(2) == 2);
    CHECK(*decode_graph_bucket(3) == 4 && *decode_graph_bucket(4) == 4 && *decode_graph_bucket(5) == 8);
    CHECK(*decode_graph_bucket(8) == 8 && *decode_graph_bucket(9) == 16 && *decode_graph_bucket(16) == 16);
    CHECK(!decode_graph_bucket(17));
    using M = BatchedDecodeMeta;
    static_assert(M::kWords == 177 && M::kMasksByteOffset == 768 && M::kBlobBytes == 816, "blob layout");
    std::vector<StepSlice> sl(3);
    for (int r = 0; r < 3; ++r) {
        sl[r].tokens = {100 + r};
        sl[r].ctx_len_before = (size_t)(15 + 16 * r);   // positions 15, 31, 47: the last slot of a page each
        sl[r].block_table = {7, 3, 9, 4};
        sl[r].state_in_slot = r;
        sl[r].state_out_slot = 10 + r;
        sl[r].has_initial_state = r != 1;
    }
    sl[2].checkpoints = {{1, 6}};
    M m;
    CHECK(pack_batched_decode_meta(sl, {0, 5}, {}, 2, 16, &m));
    const auto& w = m.words;
    CHECK(w[M::kTokenIds] == 100 && w[M::kTokenIds + 2] == 102 && w[M::kTokenIds + 3] == 0);
    CHECK(w[M::kPositions] == 15 && w[M::kPositions + 1] == 31 + 5 && w[M::kPositions + 2] == 47);
    CHECK(w[M::kWriteSlots] == 7 * 16 + 15 && w[M::kWriteSlots + 1] == 3 * 16 + 15 && w[M::kWriteSlots + 2] == 9 * 16 + 15);
    for (size_t r = 3; r < M::N; ++r) CHECK(w[M::kWriteSlots + r] == -1 && w[M::kStateOut + r] == -1 && w[M::kLoraIds + r] == -1);
    for (size_t i = 0; i <= M::N; ++i) CHECK(w[M::kQStartLoc + i] == (int32_t)i);
    CHECK(w[M::kCtxBefore + 1] == 31 && w[M::kSeqAfter + 1] == 32 && w[M::kCtxBefore + 3] == 0 && w[M::kSeqAfter + 3] == 0);
    CHECK(w[M::kStateIn + 2] == 2 && w[M::kStateOut + 2] == 12 && w[M::kCheckpointDst + 2] == 6 && w[M::kCheckpointOffset + 2] == 1);
    CHECK(w[M::kCheckpointDst] == -1 && w[M::kLoraIds] == 2 && w[M::kLoraIds + 2] == 2);
    CHECK(m.masks[M::kHasInitialState] == 1 && m.masks[M::kHasInitialState + 1] == 0 && m.masks[M::kValidReq + 2] == 1);
    CHECK(m.masks[M::kValidReq + 3] == 0 && m.masks[M::kValidToken + 2] == 1 && m.masks[M::kValidToken + 3] == 0);
    const auto blob = m.blob();
    CHECK(blob.size() == 816 && blob[M::kMasksByteOffset + M::kValidReq] == 1 && blob[4 * M::kTokenIds] == 100);
    // a decode row has one token, no speculative slots, and a table that reaches its position
    sl[0].tokens = {1, 2};
    CHECK(!pack_batched_decode_meta(sl, {}, {}, -1, 16, &m));
    sl[0].tokens = {1};
    sl[0].block_table = {};
    CHECK(!pack_batched_decode_meta(sl, {}, {}, -1, 16, &m));
    sl[0].block_table = {7};
    CHECK(pack_batched_decode_meta(sl, {}, {}, -1, 16, &m));        // position 15 is in the first page
    sl[0].ctx_len_before = 16;
    CHECK(!pack_batched_decode_meta(sl, {}, {}, -1, 16, &m));       // position 16 is not
    CHECK(pack_batched_decode_meta(sl, {}, {}, -1, 64, &m) && m.words[M::kWriteSlots] == 7 * 64 + 16);
    CHECK(!pack_batched_decode_meta({}, {}, {}, -1, 16, &m));
    CHECK(!pack_batched_decode_meta(std::vector<StepSlice>(17, sl[1]), {}, {}, -1, 16, &m));
    const warp34_attention_batch b = M::batch_at(0x10000, 0x20000, 4, 32, 8192, 0, 0.0625f);
    CHECK(b.num_reqs == 4 && b.total_tokens == 4 && b.max_q_len == 1 && b.max_blocks_per_req == 32);
    CHECK((uint64_t)(uintptr_t)b.valid_req_mask == 0x10000 + 768 + 16 && (uint64_t)(uintptr_t)b.seq_lens_after == 0x10000 + 4 * 81);
    std::puts("ok batched_decode_meta");
}

static void test_block_table_mirror() {  // graph_io.rs:886-1010
    BlockTableMirror mir(8);
    std::vector<StepSlice> sl(2);
    sl[0].block_table = {5, 6};
    sl[1].block_table = {9};
    auto sp = mir.dirty_spans(sl);
    CHECK(sp && sp->size() == 2 && (*sp)[0].row == 0 && (*sp)[0].start == 0 && (*sp)[0].entries == std::vector<int32_t>({5, 6}));
    CHECK((*sp)[1].dst_byte_offset == 8 * 4);
    sp = mir.dirty_spans(sl);
    CHECK(sp && sp->empty());                                     // nothing changed: nothing to copy
    sl[0].block_table = {5, 6, 7};                                // grew: only the tail
    sp = mir.dirty_spans(sl);
    CHECK(sp && sp->size() == 1 && (*sp)[0].start == 2 && (*sp)[0].entries == std::vector<int32_t>({7}) &&
          (*sp)[0].dst_byte_offset == 2 * 4);
    sl[1].block_table = {4, 9};                                   // another request took the row: the whole row
    sp = mir.dirty_spans(sl);
    CHECK(sp && sp->size() == 1 && (*sp)[0].row == 1 && (*sp)[0].start == 0 && (*sp)[0].entries.size() == 2);
    mir.invalidate(*sp);                                          // the copy failed: next time the whole row again
    sp = mir.dirty_spans(sl);
    CHECK(sp && sp->size() == 1 && (*sp)[0].row == 1 && (*sp)[0].start == 0);
    sp = mir.dirty_spans(sl, false);
    CHECK(sp && sp->empty());
    sl[0].block_table.assign(9, 1);
    CHECK(!mir.dirty_spans(sl));                                  // a row longer than the device row
    std::puts("ok block_table_mirror");
}

int main() {
    test_row_bytes();
    test_policy_resolution();
    test_bytes_per_token();
    test_policy_names();
    test_page_bitmap();
    test_kv_pool_layout();
    test_slot_mapping_and_step_blob();
    test_reservation_and_prefix_sharing();
    test_radix_initialization();
    test_radix_insert_exact_and_match();
    test_radix_split_and_branch();
    test_radix_dual_lock_and_eviction();
    test_radix_rollback_and_lru_order();
    test_radix_superseded_linear_turns();
    test_radix_decode_tail_leaf();
    test_radix_arena_reuse();
    test_radix_recycle_and_invalidate();
    test_radix_dual_lock_dual_lru_tombstone_and_split();
    test_radix_random_walk();
    test_spec_verify_meta();
    test_batched_decode_meta();
    test_block_table_mirror();
    std::puts("all host tests passed");
    return 0;
}
