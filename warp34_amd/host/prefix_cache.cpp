// Prefix-shared KV pages: the radix tree behind prefix hits, page eviction and the page side of
// a request's donation.  Behaviour follows crates/warp34-host/src/radix.rs (MambaRadixCache and
// the page half of ReqRadixState); the layout is this library's own: one node arena, child maps
// keyed by the first page of the child's key, and two intrusive recency lists through the arena.
// Key salting per adapter (radix.rs:400-409, 590-596) is left to the caller: token ids arrive
// here already salted.
#include <algorithm>
#include <stdexcept>

#include "kv_host.h"

namespace warp34_host {

PrefixPageCache::PrefixPageCache(size_t page_size, size_t state_chunk_tokens)
    : page_size_(page_size), chunk_(state_chunk_tokens ? state_chunk_tokens : page_size) {
    if (page_size_ == 0) throw std::invalid_argument("page_size must be > 0");
    if (chunk_ < page_size_ || chunk_ % page_size_ != 0)
        throw std::invalid_argument("state_chunk_tokens must be a multiple of page_size");
    reset();
}

void PrefixPageCache::reset() {
    nodes_.clear();
    free_ids_.clear();
    lru_head_[0] = lru_head_[1] = lru_tail_[0] = lru_tail_[1] = -1;
    full_evictable_pages_ = full_protected_pages_ = 0;
    state_evictable_slots_ = state_protected_slots_ = 0;
    nodes_.emplace_back();
    Node& root = nodes_[0];  // never evicted: both counts start at one
    root.full_lock_ref = 1;
    root.state_lock_ref = 1;
    root.alive = true;
}

// ---- arena and recency lists ------------------------------------------------------------------
int PrefixPageCache::alloc_node() {
    int id;
    if (!free_ids_.empty()) {
        id = free_ids_.back();
        free_ids_.pop_back();
        nodes_[id] = Node();
    } else {
        id = (int)nodes_.size();
        nodes_.emplace_back();
    }
    nodes_[id].alive = true;
    return id;
}

void PrefixPageCache::retire(int id) {
    Node fresh;
    nodes_[id] = fresh;  // drops key, pages and children; alive = false
    free_ids_.push_back(id);
}

void PrefixPageCache::lru_push_mru(int which, int id) {
    Node& n = nodes_[id];
    n.lru_prev[which] = lru_tail_[which];
    n.lru_next[which] = -1;
    if (lru_tail_[which] >= 0) nodes_[lru_tail_[which]].lru_next[which] = id;
    lru_tail_[which] = id;
    if (lru_head_[which] < 0) lru_head_[which] = id;
    n.in_lru[which] = true;
}

void PrefixPageCache::lru_remove(int which, int id) {
    Node& n = nodes_[id];
    if (!n.in_lru[which]) return;
    const int p = n.lru_prev[which], q = n.lru_next[which];
    if (p >= 0) nodes_[p].lru_next[which] = q; else lru_head_[which] = q;
    if (q >= 0) nodes_[q].lru_prev[which] = p; else lru_tail_[which] = p;
    n.lru_prev[which] = n.lru_next[which] = -1;
    n.in_lru[which] = false;
}

void PrefixPageCache::lru_touch(int which, int id) {
    if (id == 0) return;
    if (which == kState && !nodes_[id].has_state) return;
    lru_remove(which, id);
    lru_push_mru(which, id);
}

// page order along [node .. root), root side first, so that a child is more recent than its parent
void PrefixPageCache::touch_path(int node) {
    std::vector<int> chain;
    for (int n = node; n > 0; n = nodes_[n].parent) chain.push_back(n);
    for (auto it = chain.rbegin(); it != chain.rend(); ++it) lru_touch(kFull, *it);
}

// whole pages that key and rest have in common, counted in tokens
size_t PrefixPageCache::common_pages(const std::vector<int32_t>& key, const int32_t* rest, size_t rest_len) const {
    const size_t max_pages = std::min(key.size(), rest_len) / page_size_;
    size_t pages = 0;
    while (pages < max_pages && std::equal(key.begin() + (long)(pages * page_size_),
                                           key.begin() + (long)((pages + 1) * page_size_), rest + pages * page_size_))
        ++pages;
    return pages * page_size_;
}

// The first split_tokens tokens of `child` move into a new node between it and its parent.  The
// new node has no snapshot (a state cannot be cut in the middle of a node) and inherits the page
// lock count, because every lock on the child runs through it (radix.rs:306-378).
int PrefixPageCache::split_node(int child, size_t split_tokens) {
    const size_t split_pages = split_tokens / page_size_;
    const int parent = nodes_[child].parent;
    const int mid = alloc_node();
    Node& c = nodes_[child];
    Node& m = nodes_[mid];
    m.parent = parent;
    m.key.assign(c.key.begin(), c.key.begin() + (long)split_tokens);
    m.pages.assign(c.pages.begin(), c.pages.begin() + (long)split_pages);
    if (c.draft_pages.size() >= split_pages) {
        m.draft_pages.assign(c.draft_pages.begin(), c.draft_pages.begin() + (long)split_pages);
        c.draft_pages.erase(c.draft_pages.begin(), c.draft_pages.begin() + (long)split_pages);
    } else {
        c.draft_pages.clear();
    }
    m.full_lock_ref = c.full_lock_ref;
    c.key.erase(c.key.begin(), c.key.begin() + (long)split_tokens);
    c.pages.erase(c.pages.begin(), c.pages.begin() + (long)split_pages);
    c.parent = mid;
    m.children.emplace(std::vector<int32_t>(c.key.begin(), c.key.begin() + (long)page_size_), child);
    nodes_[parent].children[std::vector<int32_t>(m.key.begin(), m.key.begin() + (long)page_size_)] = mid;
    // both halves become the most recent entries of the page order, parent half first
    lru_remove(kFull, child);
    lru_push_mru(kFull, mid);
    lru_push_mru(kFull, child);
    return mid;
}

// ---- lookups ------------------------------------------------------------------------------------
PrefixMatch PrefixPageCache::match_prefix(const std::vector<int32_t>& token_ids) {
    ++total_lookups;
    total_lookup_tokens += token_ids.size();
    PrefixMatch m;
    const size_t aligned = (token_ids.size() / page_size_) * page_size_;
    if (disable || aligned == 0) return m;

    std::vector<int> path;
    int cur = 0;
    size_t off = 0;
    while (off < aligned) {
        const std::vector<int32_t> first(token_ids.begin() + (long)off, token_ids.begin() + (long)(off + page_size_));
        const auto it = nodes_[cur].children.find(first);
        if (it == nodes_[cur].children.end()) break;
        const int child = it->second;
        const size_t common = common_pages(nodes_[child].key, token_ids.data() + off, aligned - off);
        if (common < nodes_[child].key.size()) {  // the query leaves this node half way: cut it there
            path.push_back(split_node(child, common));
            break;
        }
        path.push_back(child);
        cur = child;
        off += common;
    }
    // the usable part ends at the deepest node that still has a snapshot
    size_t best_len = 0;
    int best = 0;
    for (size_t i = 0; i < path.size(); ++i) {
        if (nodes_[path[i]].has_state) {
            best_len = i + 1;
            best = path[i];
        }
    }
    touch_path(best);
    lru_touch(kState, best);

    for (size_t i = 0; i < path.size(); ++i) m.kv_matched_tokens += nodes_[path[i]].key.size();
    for (size_t i = 0; i < best_len; ++i) {
        Node& n = nodes_[path[i]];
        n.decode_tail = false;  // somebody continued from here: the tokens are verified
        m.kv_pages.insert(m.kv_pages.end(), n.pages.begin(), n.pages.end());
        m.draft_pages.insert(m.draft_pages.end(), n.draft_pages.begin(), n.draft_pages.end());
    }
    m.matched_tokens = m.kv_pages.size() * page_size_;
    m.has_state = best != 0 && nodes_[best].has_state;
    m.state_slot = m.has_state ? nodes_[best].state_slot : -1;
    m.last_node = best;
    if (path.size() > best_len) m.state_branching_seqlen = (m.kv_matched_tokens / chunk_) * chunk_;
    total_hit_tokens += m.matched_tokens;
    if (m.has_state) ++total_state_hits;
    return m;
}

std::vector<int32_t> PrefixPageCache::collect_node_kv_pages(int node) const {
    std::vector<int> chain;
    for (int n = node; n > 0; n = nodes_[n].parent) chain.push_back(n);
    std::vector<int32_t> pages;
    for (auto it = chain.rbegin(); it != chain.rend(); ++it)
        pages.insert(pages.end(), nodes_[*it].pages.begin(), nodes_[*it].pages.end());
    return pages;
}

// ---- locks ----------------------------------------------------------------------------------------
void PrefixPageCache::inc_lock_ref(int node) {
    if (disable || node == 0) return;
    Node& n = nodes_[node];
    if (n.has_state) {
        if (n.state_lock_ref == 0) {
            state_evictable_slots_ -= state_evictable_slots_ ? 1 : 0;
            ++state_protected_slots_;
        }
        ++n.state_lock_ref;
    }
    for (int cur = node; cur > 0; cur = nodes_[cur].parent) {
        Node& c = nodes_[cur];
        if (c.full_lock_ref == 0) {
            full_evictable_pages_ -= std::min(full_evictable_pages_, c.pages.size());
            full_protected_pages_ += c.pages.size();
        }
        ++c.full_lock_ref;
    }
}

void PrefixPageCache::dec_lock_ref(int node) {
    if (disable || node == 0) return;
    Node& n = nodes_[node];
    if (n.has_state) {
        if (n.state_lock_ref == 0) throw std::logic_error("dec_lock_ref: snapshot lock count is zero");
        if (n.state_lock_ref == 1) {
            ++state_evictable_slots_;
            state_protected_slots_ -= state_protected_slots_ ? 1 : 0;
        }
        --n.state_lock_ref;
    }
    for (int cur = node; cur > 0; cur = nodes_[cur].parent) {
        Node& c = nodes_[cur];
        if (c.full_lock_ref == 0) throw std::logic_error("dec_lock_ref: page lock count is zero");
        if (c.full_lock_ref == 1) {
            full_evictable_pages_ += c.pages.size();
            full_protected_pages_ -= std::min(full_protected_pages_, c.pages.size());
        }
        --c.full_lock_ref;
    }
}

// ---- insert ---------------------------------------------------------------------------------------
PrefixInsertResult PrefixPageCache::insert(const std::vector<int32_t>& token_ids, const std::vector<int32_t>& kv_pages,
                                           const std::vector<int32_t>& draft_pages, int32_t state_slot,
                                           size_t prev_protected_pages) {
    if (token_ids.size() % page_size_ != 0) throw std::invalid_argument("insert: token count is not page-aligned");
    if (token_ids.size() / page_size_ != kv_pages.size())
        throw std::invalid_argument("insert: one page per page_size tokens expected");
    if (!draft_pages.empty() && draft_pages.size() != kv_pages.size())
        throw std::invalid_argument("insert: draft pages must be absent or match the pages");
    PrefixInsertResult r;
    if (disable || token_ids.empty()) {
        r.state_already_existed = true;
        return r;
    }
    int cur = 0;
    size_t off = 0, page_off = 0;
    while (off < token_ids.size()) {
        const std::vector<int32_t> first(token_ids.begin() + (long)off, token_ids.begin() + (long)(off + page_size_));
        const auto it = nodes_[cur].children.find(first);
        if (it == nodes_[cur].children.end()) break;
        const int child = it->second;
        lru_touch(kFull, child);
        const size_t common = common_pages(nodes_[child].key, token_ids.data() + off, token_ids.size() - off);
        const size_t common_pg = common / page_size_;
        // the caller's pages over this stretch are copies of the tree's, except the leading ones it
        // borrowed from the tree in the first place
        if (prev_protected_pages < page_off + common_pg) {
            const size_t start = prev_protected_pages > page_off ? prev_protected_pages - page_off : 0;
            r.freed_duplicate_kv_pages.insert(r.freed_duplicate_kv_pages.end(),
                                              kv_pages.begin() + (long)(page_off + start),
                                              kv_pages.begin() + (long)(page_off + common_pg));
            if (!draft_pages.empty())
                r.freed_duplicate_draft_pages.insert(r.freed_duplicate_draft_pages.end(),
                                                     draft_pages.begin() + (long)(page_off + start),
                                                     draft_pages.begin() + (long)(page_off + common_pg));
        }
        off += common;
        page_off += common_pg;
        if (common < nodes_[child].key.size()) {
            cur = split_node(child, common);
            break;
        }
        nodes_[child].decode_tail = false;
        cur = child;
    }

    if (off < token_ids.size()) {  // a new leaf with the rest
        const int leaf = alloc_node();
        Node& n = nodes_[leaf];
        n.parent = cur;
        n.key.assign(token_ids.begin() + (long)off, token_ids.end());
        n.pages.assign(kv_pages.begin() + (long)page_off, kv_pages.end());
        if (!draft_pages.empty()) n.draft_pages.assign(draft_pages.begin() + (long)page_off, draft_pages.end());
        n.has_state = true;
        n.state_slot = state_slot;
        nodes_[cur].children.emplace(std::vector<int32_t>(n.key.begin(), n.key.begin() + (long)page_size_), leaf);
        lru_push_mru(kFull, leaf);
        lru_push_mru(kState, leaf);
        full_evictable_pages_ += n.pages.size();
        ++state_evictable_slots_;
        r.terminal_node = leaf;
    } else if (!nodes_[cur].has_state) {  // the sequence ends on a tombstone: it takes the snapshot
        nodes_[cur].has_state = true;
        nodes_[cur].state_slot = state_slot;
        lru_touch(kFull, cur);
        lru_push_mru(kState, cur);
        ++state_evictable_slots_;
        r.terminal_node = cur;
    } else {
        r.state_already_existed = true;
        lru_touch(kFull, cur);
        r.terminal_node = cur;
    }
    r.existing_prefix_tokens = off;
    return r;
}

// ---- eviction -------------------------------------------------------------------------------------
// Removes an unlocked leaf; ancestors that are left as unlocked, snapshot-less leaves go with it
// (radix.rs:701-756).  Pages are reported leaf first.
void PrefixPageCache::delete_leaf(int leaf, EvictResult* out) {
    Node& l = nodes_[leaf];
    if (l.full_lock_ref != 0 || l.state_lock_ref != 0 || !l.children.empty() || !l.has_state)
        throw std::logic_error("delete_leaf: node is locked, internal or a tombstone");
    out->freed_kv_pages.insert(out->freed_kv_pages.end(), l.pages.begin(), l.pages.end());
    out->freed_draft_pages.insert(out->freed_draft_pages.end(), l.draft_pages.begin(), l.draft_pages.end());
    out->freed_state_slots.push_back(l.state_slot);
    state_evictable_slots_ -= state_evictable_slots_ ? 1 : 0;
    full_evictable_pages_ -= std::min(full_evictable_pages_, l.pages.size());
    lru_remove(kFull, leaf);
    lru_remove(kState, leaf);
    int parent = l.parent;
    nodes_[parent].children.erase(std::vector<int32_t>(l.key.begin(), l.key.begin() + (long)page_size_));
    retire(leaf);
    while (parent != 0) {
        Node& p = nodes_[parent];
        if (!p.children.empty() || p.has_state || p.full_lock_ref > 0) break;
        out->freed_kv_pages.insert(out->freed_kv_pages.end(), p.pages.begin(), p.pages.end());
        out->freed_draft_pages.insert(out->freed_draft_pages.end(), p.draft_pages.begin(), p.draft_pages.end());
        full_evictable_pages_ -= std::min(full_evictable_pages_, p.pages.size());
        lru_remove(kFull, parent);
        const int grand = p.parent;
        nodes_[grand].children.erase(std::vector<int32_t>(p.key.begin(), p.key.begin() + (long)page_size_));
        retire(parent);
        parent = grand;
    }
}

EvictResult PrefixPageCache::evict_full_pages(size_t num_pages) {
    EvictResult out;
    if (disable || num_pages == 0) return out;
    auto evictable_leaf = [&](const Node& n) {
        return n.children.empty() && n.full_lock_ref == 0 && n.state_lock_ref == 0;
    };
    while (out.freed_kv_pages.size() < num_pages) {
        int victim = -1;
        for (int id = lru_head_[kFull]; id >= 0; id = nodes_[id].lru_next[kFull]) {
            if (evictable_leaf(nodes_[id]) && nodes_[id].decode_tail) {
                victim = id;
                break;
            }
        }
        if (victim < 0) {
            for (int id = lru_head_[kFull]; id >= 0; id = nodes_[id].lru_next[kFull]) {
                if (evictable_leaf(nodes_[id])) {
                    victim = id;
                    break;
                }
            }
        }
        if (victim < 0) break;
        delete_leaf(victim, &out);
    }
    return out;
}

void PrefixPageCache::mark_node_decode_tail(int node) {
    if (node != 0 && nodes_[node].children.empty()) nodes_[node].decode_tail = true;
}

// a snapshot of verified tokens somewhere below `node` (radix.rs:778-789)
bool PrefixPageCache::has_verified_state_below(int node) const {
    for (const auto& kv : nodes_[node].children) {
        const Node& c = nodes_[kv.second];
        if ((c.has_state && !c.decode_tail) || has_verified_state_below(kv.second)) return true;
    }
    return false;
}

// An internal node whose snapshot a longer verified one has overtaken, on a path that does not
// fork into verified branches (radix.rs:791-811): taking its snapshot costs no page and no hit.
bool PrefixPageCache::superseded_linear_internal(int node) const {
    const Node& n = nodes_[node];
    if (n.state_lock_ref > 0 || n.children.empty() || !has_verified_state_below(node)) return false;
    size_t verified_children = 0;
    for (const auto& kv : n.children) {
        const Node& c = nodes_[kv.second];
        if (!(c.children.empty() && c.decode_tail)) ++verified_children;
    }
    return verified_children == 1;
}

// An unlocked decode-tail leaf below a prompt that keeps a snapshot of its own (radix.rs:813-835).
bool PrefixPageCache::reclaimable_decode_tail_leaf(int node) const {
    const Node& n = nodes_[node];
    if (!n.children.empty() || !n.decode_tail || n.full_lock_ref > 0 || n.state_lock_ref > 0) return false;
    for (int p = n.parent; p > 0; p = nodes_[p].parent)
        if (nodes_[p].has_state || has_verified_state_below(p)) return true;
    return false;
}

bool PrefixPageCache::has_evictable_internal_state() const {
    if (disable) return false;
    for (int id = lru_head_[kState]; id >= 0; id = nodes_[id].lru_next[kState])
        if (superseded_linear_internal(id) || reclaimable_decode_tail_leaf(id)) return true;
    return false;
}

EvictResult PrefixPageCache::evict_state_slots(size_t num_slots) {
    EvictResult out;
    if (disable || num_slots == 0) return out;
    while (out.freed_state_slots.size() < num_slots) {
        int victim = -1;
        for (int id = lru_head_[kState]; id >= 0 && victim < 0; id = nodes_[id].lru_next[kState])
            if (superseded_linear_internal(id)) victim = id;
        for (int id = lru_head_[kState]; id >= 0 && victim < 0; id = nodes_[id].lru_next[kState])
            if (reclaimable_decode_tail_leaf(id)) victim = id;
        for (int id = lru_head_[kState]; id >= 0 && victim < 0; id = nodes_[id].lru_next[kState]) {
            const Node& n = nodes_[id];
            if (n.state_lock_ref == 0 && (!n.children.empty() || n.full_lock_ref == 0)) victim = id;
        }
        if (victim < 0) break;
        Node& v = nodes_[victim];
        if (!v.children.empty()) {  // internal: the pages stay for the descendants
            out.freed_state_slots.push_back(v.state_slot);
            v.has_state = false;
            v.state_slot = -1;
            state_evictable_slots_ -= state_evictable_slots_ ? 1 : 0;
            lru_remove(kState, victim);
        } else {
            delete_leaf(victim, &out);
        }
    }
    return out;
}

EvictResult PrefixPageCache::invalidate_state_slot(int32_t slot) {
    EvictResult out;
    if (disable) return out;
    std::vector<int> holders;
    for (size_t i = 1; i < nodes_.size(); ++i)
        if (nodes_[i].alive && nodes_[i].has_state && nodes_[i].state_slot == slot) holders.push_back((int)i);
    for (int id : holders) {
        Node& n = nodes_[id];
        if (!n.alive) continue;  // went with an earlier holder's clean-up
        if (!n.children.empty() || n.full_lock_ref > 0) {
            n.has_state = false;
            n.state_slot = -1;
            if (n.state_lock_ref == 0) {
                state_evictable_slots_ -= state_evictable_slots_ ? 1 : 0;
                lru_remove(kState, id);
            }
        } else {
            delete_leaf(id, &out);
            out.freed_state_slots.erase(std::remove(out.freed_state_slots.begin(), out.freed_state_slots.end(), slot),
                                        out.freed_state_slots.end());
        }
    }
    return out;
}

bool PrefixPageCache::can_recycle_locked_state(int node) const {
    if (disable || node == 0) return false;
    return nodes_[node].state_lock_ref == 1 && nodes_[node].has_state;
}

int32_t PrefixPageCache::reclaim_internal_state(int node) {
    if (disable || node == 0) return -1;
    Node& n = nodes_[node];
    if (n.state_lock_ref > 0 || n.children.empty() || !n.has_state) return -1;
    const int32_t slot = n.state_slot;
    n.has_state = false;
    n.state_slot = -1;
    state_evictable_slots_ -= state_evictable_slots_ ? 1 : 0;
    lru_remove(kState, node);
    return slot;
}

void PrefixPageCache::set_node_state(int node, int32_t slot) {
    if (node == 0 || !node_alive(node)) throw std::invalid_argument("set_node_state: no such node");
    Node& n = nodes_[node];
    if (!n.has_state) {
        n.has_state = true;
        lru_push_mru(kState, node);
        if (n.state_lock_ref == 0) ++state_evictable_slots_; else ++state_protected_slots_;
    }
    n.state_slot = slot;
}

bool PrefixPageCache::sanity_check(std::string* why) const {
    auto fail = [&](const std::string& msg) {
        if (why) *why = msg;
        return false;
    };
    size_t ev_pages = 0, pr_pages = 0, ev_state = 0, pr_state = 0, in_full = 0, in_state = 0;
    for (size_t i = 1; i < nodes_.size(); ++i) {
        const Node& n = nodes_[i];
        if (!n.alive) continue;
        const std::string tag = "node " + std::to_string(i);
        if (n.full_lock_ref < n.state_lock_ref) return fail(tag + ": page lock count below snapshot lock count");
        if (n.children.empty() && !n.has_state && n.full_lock_ref == 0) return fail(tag + ": unlocked tombstone leaf");
        if (n.key.size() != n.pages.size() * page_size_ || n.pages.empty()) return fail(tag + ": key / pages mismatch");
        if (!n.in_lru[kFull]) return fail(tag + ": missing from the page order");
        if (n.in_lru[kState] != n.has_state) return fail(tag + ": snapshot order membership");
        (n.full_lock_ref == 0 ? ev_pages : pr_pages) += n.pages.size();
        if (n.has_state) ++(n.state_lock_ref == 0 ? ev_state : pr_state);
        for (const auto& kv : n.children)
            if (nodes_[kv.second].parent != (int)i || !nodes_[kv.second].alive) return fail(tag + ": child link");
    }
    for (int which = 0; which < 2; ++which) {
        int prev = -1;
        size_t count = 0;
        for (int id = lru_head_[which]; id >= 0; id = nodes_[id].lru_next[which]) {
            if (!nodes_[id].alive || nodes_[id].lru_prev[which] != prev) return fail("recency list links");
            prev = id;
            if (++count > nodes_.size()) return fail("recency list cycle");
        }
        if (prev != lru_tail_[which]) return fail("recency list tail");
        (which == kFull ? in_full : in_state) = count;
    }
    size_t alive = 0, with_state = 0;
    for (size_t i = 1; i < nodes_.size(); ++i) {
        alive += nodes_[i].alive;
        with_state += nodes_[i].alive && nodes_[i].has_state;
    }
    if (in_full != alive || in_state != with_state) return fail("recency list length");
    if (ev_pages != full_evictable_pages_) return fail("full_evictable_pages: tracked " + std::to_string(full_evictable_pages_) + " actual " + std::to_string(ev_pages));
    if (pr_pages != full_protected_pages_) return fail("full_protected_pages: tracked " + std::to_string(full_protected_pages_) + " actual " + std::to_string(pr_pages));
    if (ev_state != state_evictable_slots_) return fail("state_evictable_slots: tracked " + std::to_string(state_evictable_slots_) + " actual " + std::to_string(ev_state));
    if (pr_state != state_protected_slots_) return fail("state_protected_slots: tracked " + std::to_string(state_protected_slots_) + " actual " + std::to_string(pr_state));
    return true;
}

// ---- a request's pages ------------------------------------------------------------------------------
void RequestPages::restore_prefix_hit(PrefixPageCache& cache, const std::vector<int32_t>& prompt_tokens,
                                      const PrefixMatch& m) {
    if (!m.has_state || m.matched_tokens == 0) return;
    cache.inc_lock_ref(m.last_node);
    token_ids.assign(prompt_tokens.begin(), prompt_tokens.begin() + (long)m.matched_tokens);
    kv_pages = m.kv_pages;
    draft_pages = m.draft_pages;
    protected_pages = kv_pages.size();
    last_locked_node = m.last_node;
    page_size = cache.page_size();
}

std::vector<int32_t> RequestPages::rollback_uncommitted_kv_pages() {
    size_t needed = page_size ? (token_ids.size() + page_size - 1) / page_size : kv_pages.size();
    needed = std::max(needed, protected_pages);
    std::vector<int32_t> freed;
    if (kv_pages.size() > needed) {
        freed.assign(kv_pages.begin() + (long)needed, kv_pages.end());
        kv_pages.resize(needed);
    }
    return freed;
}

RequestPages::Donation RequestPages::donate_pages(PrefixPageCache& cache, size_t cache_len, int32_t state_slot,
                                                  bool finish_req) {
    Donation d;
    if (page_size == 0) page_size = cache.page_size();
    const bool donatable = cache_len > protected_pages * page_size && cache_len <= token_ids.size() &&
                           cache_len % page_size == 0 && kv_pages.size() >= cache_len / page_size;
    if (donatable) {
        const size_t cache_pages = cache_len / page_size;
        const bool had_protected_prompt = protected_pages > 0;
        const std::vector<int32_t> toks(token_ids.begin(), token_ids.begin() + (long)cache_len);
        const std::vector<int32_t> pages(kv_pages.begin(), kv_pages.begin() + (long)cache_pages);
        std::vector<int32_t> drafts;
        if (draft_pages.size() >= cache_pages) drafts.assign(draft_pages.begin(), draft_pages.begin() + (long)cache_pages);
        const PrefixInsertResult ins = cache.insert(toks, pages, drafts, state_slot, protected_pages);
        if (finish_req && had_protected_prompt && !ins.state_already_existed) cache.mark_node_decode_tail(ins.terminal_node);
        d.donated_seq_len = cache_len;
        d.state_already_existed = ins.state_already_existed;
        d.freed_kv_pages = ins.freed_duplicate_kv_pages;
        d.freed_draft_pages = ins.freed_duplicate_draft_pages;
        // where the tree had the tokens already, the request goes on with the tree's pages
        const std::vector<int32_t> canonical = cache.collect_node_kv_pages(ins.terminal_node);
        if (canonical.size() == cache_pages) std::copy(canonical.begin(), canonical.end(), kv_pages.begin());
        cache.dec_lock_ref(last_locked_node);
        if (finish_req) {
            last_locked_node = 0;
        } else {
            cache.inc_lock_ref(ins.terminal_node);
            last_locked_node = ins.terminal_node;
        }
        protected_pages = cache_pages;
    } else if (finish_req) {
        cache.dec_lock_ref(last_locked_node);
        last_locked_node = 0;
    }
    if (finish_req) {
        if (kv_pages.size() > protected_pages)
            d.freed_kv_pages.insert(d.freed_kv_pages.end(), kv_pages.begin() + (long)protected_pages, kv_pages.end());
        if (draft_pages.size() > protected_pages)
            d.freed_draft_pages.insert(d.freed_draft_pages.end(), draft_pages.begin() + (long)protected_pages,
                                       draft_pages.end());
    }
    return d;
}

}  // namespace warp34_host
