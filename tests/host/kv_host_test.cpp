// Host-logic tests; cases follow the reference's own unit tests
// (crates/warp34-host/src/cache.rs:628-826, model/graph_io.rs:1286) plus the page-reservation
// and prefix-sharing behaviour of model/batch.rs:57-93 and radix.rs:1129-1157,1234-1245.
// Prints one "ok <name>" line per passing test; exits non-zero at the first failure.
#include <cstdio>
#include <cstdlib>
#include <set>

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

static void test_reservation_and_prefix_sharing() {
    HostAllocator ha;
    KvPool pool;
    CHECK(!KvPool::new_target_full_attn(&pool, ha, 0, {0}, 2, 256, 16, 12, KvFormatPolicy::Tq4All, false));
    PrefixPageCache cache(16);

    // request A: 70 tokens -> 5 pages, ascending page ids
    RequestPages a;
    a.page_size = 16;
    CHECK(reserve_kv_pages_from(pool, cache, &a.kv_pages, 5));
    CHECK((a.kv_pages == std::vector<int32_t>{0, 1, 2, 3, 4}));
    CHECK(reserve_kv_pages_from(pool, cache, &a.kv_pages, 3));  // already satisfied
    a.token_ids = iota_tokens(70, 1);
    // A finishes: its four whole pages are donated, the partial fifth goes back to the pool
    std::vector<int32_t> dup;
    const int node_a = cache.insert(a.token_ids, a.kv_pages, &dup);
    CHECK(dup.empty() && node_a != 0 && cache.cached_pages() == 4);
    pool.free_page(a.kv_pages[4]);
    CHECK(pool.free_count() == 8 && cache.full_evictable_pages() == 4);

    // request B shares the first 40 tokens of A -> two whole pages hit
    std::vector<int32_t> prompt_b = iota_tokens(40, 1);
    for (int i = 0; i < 30; ++i) prompt_b.push_back(900000 + i);
    const PrefixMatch mb = cache.match_prefix(prompt_b);
    CHECK(mb.matched_tokens == 32 && (mb.kv_pages == std::vector<int32_t>{0, 1}));
    RequestPages b;
    b.restore_prefix_hit(cache, prompt_b, mb);
    CHECK(b.protected_pages == 2 && b.token_ids.size() == 32 && cache.full_protected_pages() == 2);
    // B needs ceil(70/16) = 5 pages: three private ones, lowest free ids first
    CHECK(reserve_kv_pages_from(pool, cache, &b.kv_pages, 5));
    CHECK((b.kv_pages == std::vector<int32_t>{0, 1, 4, 5, 6}));

    // speculative tail: B reserves two more pages, commits only up to 85 tokens, rolls back
    b.token_ids = prompt_b;
    CHECK(reserve_kv_pages_from(pool, cache, &b.kv_pages, 7));
    b.token_ids.resize(70);
    for (int i = 0; i < 15; ++i) b.token_ids.push_back(i);
    const std::vector<int32_t> rolled = b.rollback_uncommitted_kv_pages();
    CHECK((rolled == std::vector<int32_t>{8}) && b.kv_pages.size() == 5 + 1);
    free_kv_pages(pool, rolled);
    // rollback never drops a shared page even when nothing is committed
    RequestPages c = b;
    c.token_ids.clear();
    const std::vector<int32_t> rolled_c = c.rollback_uncommitted_kv_pages();
    CHECK(c.kv_pages.size() == 2 && rolled_c.size() == 4);

    // pool pressure: 12 pages, cache holds 0..3 (0 and 1 locked), B holds 4,5,6,7 -> free 8..11
    CHECK(pool.free_count() == 4);
    std::vector<int32_t> big;
    CHECK(reserve_kv_pages_from(pool, cache, &big, 6));  // evicts the two unlocked cached pages
    CHECK(cache.cached_pages() == 2 && cache.full_evictable_pages() == 0);
    CHECK((big == std::vector<int32_t>{2, 3, 8, 9, 10, 11}));
    std::vector<int32_t> more;
    CHECK(!reserve_kv_pages_from(pool, cache, &more, 1));  // locked pages cannot be evicted
    CHECK(more.empty());
    cache.dec_lock_ref(b.last_locked_node);
    CHECK(reserve_kv_pages_from(pool, cache, &more, 2));
    CHECK((more == std::vector<int32_t>{0, 1}) && cache.cached_pages() == 0);

    // duplicate donation: same tokens under other physical pages are handed back
    PrefixPageCache c2(16);
    const std::vector<int32_t> t = iota_tokens(32, 7);
    c2.insert(t, {20, 21}, nullptr);
    std::vector<int32_t> d2;
    c2.insert(t, {30, 21}, &d2);
    CHECK((d2 == std::vector<int32_t>{30}) && c2.cached_pages() == 2);
    std::puts("ok reservation_and_prefix_sharing");
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
    std::puts("all host tests passed");
    return 0;
}
