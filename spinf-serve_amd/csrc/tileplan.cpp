// Tile-plan compiler: stream metadata -> per-query-tile list of visible key tiles with 32x32 activity / mask bits.
// Stands in for block_tables (spinf_serve/packer.py:426-491); the visibility predicate is the one of
// spinf_serve/scorer.py:173-177, with the image groups of scorer.py:184-198 (the tokens of a group also see each other both
// ways).  Host code, no global state.
#include "spinf_tree.h"
#include "common.h"

#include <algorithm>
#include <cstring>
#include <new>
#include <unordered_map>
#include <vector>

struct spinf_tileplan {
    int64_t n = 0;
    int32_t window = 0;
    int32_t ktile = SPINF_KTILE;     // keys per entry: 64, or 32 for the head dim 512 kernel (one sub-tile per entry)
    std::vector<int32_t> qt_ptr, kv_idx, order;
    std::vector<uint32_t> kv_bits;
    std::vector<int64_t> weight;     // cost of a query tile in 32 x 32 blocks: per key tile, 4 x the most blocks any row group sees
    std::vector<int32_t> group;      // job of the tile's first real row (-1: pads only)
    int64_t active = 0, masked = 0;
};

namespace {

struct Blk {            // aggregates of one 32-token block
    int32_t lo, hi;     // token range [lo, hi)
    bool all_real;      // every token is a real token
    int32_t job;        // the single job of its tokens, -2 if mixed / pads present
    int32_t min_end, max_end;   // over all tokens (pads count as -1)
    int64_t min_pos, max_pos;   // over real tokens
    bool any_real;
};

// grp_mode 1: the group term holds past the window; 2: it is windowed like the rest (scorer.py:186-198)
inline bool visible(const int32_t* art, const int32_t* end, const int32_t* pos, const int32_t* grp, int32_t grp_mode, int32_t window,
                    int64_t q, int64_t k) {
    if (q == k) return true;
    const bool in_window = window <= 0 || ((int64_t)pos[q] - (int64_t)pos[k]) < (int64_t)window;
    const bool v = k <= q && art[q] >= 0 && art[k] == art[q] && q < (int64_t)end[k] && in_window;
    if (v || !grp) return v;
    return grp[q] >= 0 && grp[q] == grp[k] && (grp_mode == 1 || in_window);
}

// do two sorted lists share a value?
inline bool share(const std::vector<int32_t>& a, const std::vector<int32_t>& b) {
    size_t i = 0, j = 0;
    while (i < a.size() && j < b.size()) {
        if (a[i] == b[j]) return true;
        if (a[i] < b[j]) i++; else j++;
    }
    return false;
}

}  // namespace

extern "C" int spinf_tileplan_build(const int32_t* art, const int32_t* end, const int32_t* pos, int64_t n, int32_t window,
                                    spinf_tileplan** out) {
    return spinf_tileplan_build_ktile(art, end, pos, nullptr, 0, n, window, SPINF_KTILE, out);
}

extern "C" int spinf_tileplan_build_groups(const int32_t* art, const int32_t* end, const int32_t* pos, const int32_t* grp, int32_t grp_mode,
                                           int64_t n, int32_t window, spinf_tileplan** out) {
    return spinf_tileplan_build_ktile(art, end, pos, grp, grp_mode, n, window, SPINF_KTILE, out);
}

extern "C" int spinf_tileplan_build_ktile(const int32_t* art, const int32_t* end, const int32_t* pos, const int32_t* grp, int32_t grp_mode,
                                          int64_t n, int32_t window, int32_t ktile, spinf_tileplan** out) {
    if (!out) return spinf_fail(SPINF_E_ARG, "tileplan_build: out is null");
    *out = nullptr;
    if (ktile != SPINF_KTILE && ktile != SPINF_SUB) return spinf_fail(SPINF_E_ARG, "tileplan_build: key tile %d not in {64, 32}", ktile);
    if (n < 0 || (n > 0 && (!art || !end || !pos))) return spinf_fail(SPINF_E_ARG, "tileplan_build: null metadata");
    if (grp && grp_mode != 1 && grp_mode != 2) return spinf_fail(SPINF_E_ARG, "tileplan_build: group mode %d not in {1, 2}", grp_mode);
    if (n > (int64_t)1 << 30) return spinf_fail(SPINF_E_ARG, "tileplan_build: stream too long");
    spinf_tileplan* p = new (std::nothrow) spinf_tileplan;
    if (!p) return spinf_fail(SPINF_E_NOMEM, "tileplan_build: out of memory");
    try {
        p->n = n;
        p->ktile = ktile;
        p->window = window > 0 ? window : 0;
        const int32_t W = p->window;
        const int64_t nqt = (n + SPINF_QTILE - 1) / SPINF_QTILE;
        const int64_t nb = (n + SPINF_SUB - 1) / SPINF_SUB;
        std::vector<Blk> blk(nb);
        for (int64_t b = 0; b < nb; b++) {
            Blk& B = blk[b];
            B.lo = (int32_t)(b * SPINF_SUB);
            B.hi = (int32_t)std::min<int64_t>(n, (b + 1) * SPINF_SUB);
            B.all_real = true; B.any_real = false; B.job = -3;
            B.min_end = INT32_MAX; B.max_end = INT32_MIN; B.min_pos = INT64_MAX; B.max_pos = INT64_MIN;
            for (int32_t i = B.lo; i < B.hi; i++) {
                const bool real = art[i] >= 0;
                B.all_real &= real;
                B.min_end = std::min(B.min_end, end[i]);
                B.max_end = std::max(B.max_end, end[i]);
                if (real) {
                    B.any_real = true;
                    B.min_pos = std::min<int64_t>(B.min_pos, pos[i]);
                    B.max_pos = std::max<int64_t>(B.max_pos, pos[i]);
                    if (B.job == -3) B.job = art[i]; else if (B.job != art[i]) B.job = -2;
                } else {
                    B.job = -2;
                }
            }
            if (B.job == -3) B.job = -2;
        }
        // image groups: the distinct groups of every block (sorted), the last position of every group
        std::vector<std::vector<int32_t>> bgrp(grp ? nb : 0);
        std::unordered_map<int32_t, int64_t> glast;
        if (grp) {
            for (int64_t i = 0; i < n; i++) {
                if (grp[i] < 0) continue;
                std::vector<int32_t>& g = bgrp[i / SPINF_SUB];
                if (std::find(g.begin(), g.end(), grp[i]) == g.end()) g.push_back(grp[i]);
                glast[grp[i]] = i;
            }
            for (auto& g : bgrp) std::sort(g.begin(), g.end());
        }
        // first stream position of every job: the lowest key any of its rows may see
        std::unordered_map<int32_t, int64_t> first;
        std::vector<int64_t> jfirst(n);
        for (int64_t i = 0; i < n; i++) {
            if (art[i] < 0) { jfirst[i] = i; continue; }
            auto it = first.find(art[i]);
            if (it == first.end()) it = first.emplace(art[i], i).first;
            jfirst[i] = it->second;
        }
        p->qt_ptr.assign(nqt + 1, 0);
        std::vector<int64_t>& weight = p->weight;
        std::vector<int32_t>& group = p->group;
        weight.assign(nqt, 0);
        group.assign(nqt, -1);
        for (int64_t t = 0; t < nqt; t++) {
            const int64_t q0 = t * SPINF_QTILE, q1 = std::min<int64_t>(n, q0 + SPINF_QTILE);
            int64_t lo_key = q0, hi_key = q1;   // keys [lo_key, hi_key) can matter: the rows' jobs so far, and their groups to the end
            for (int64_t q = q0; q < q1; q++) {
                lo_key = std::min(lo_key, jfirst[q]);
                if (group[t] < 0 && art[q] >= 0) group[t] = art[q];
                if (grp && grp[q] >= 0) hi_key = std::max(hi_key, glast[grp[q]] + 1);
            }
            for (int64_t j = lo_key / ktile; j * ktile < hi_key; j++) {
                uint32_t bits = 0;
                for (int w = 0; w < SPINF_QTILE / SPINF_SUB; w++) {
                    const int64_t rb = q0 / SPINF_SUB + w;
                    if (rb >= nb) break;
                    const Blk& R = blk[rb];
                    for (int s = 0; s < ktile / SPINF_SUB; s++) {
                        const int64_t kb = j * (ktile / SPINF_SUB) + s;
                        if (kb >= nb) break;
                        const Blk& K = blk[kb];
                        const bool grouped = grp && share(bgrp[rb], bgrp[kb]);   // some row and some key are of one image
                        if (K.lo > R.hi - 1 && !grouped) continue;           // every key after every row
                        const bool below = K.hi - 1 < R.lo;                  // every key strictly before every row
                        bool any, all;
                        if (grouped) {
                            any = false; all = (R.hi - R.lo) == SPINF_SUB && (K.hi - K.lo) == SPINF_SUB;
                            for (int64_t q = R.lo; q < R.hi; q++)
                                for (int64_t k = K.lo; k < K.hi; k++) {
                                    const bool v = visible(art, end, pos, grp, grp_mode, W, q, k);
                                    any |= v; all &= v;
                                }
                        } else if (below && K.max_end <= R.lo) { any = false; all = false; }
                        else if (below && W > 0 && R.any_real && K.any_real && R.min_pos - K.max_pos >= W) { any = false; all = false; }
                        else if (K.hi - 1 <= R.lo && R.all_real && K.all_real && R.job >= 0 && R.job == K.job && K.min_end >= R.hi &&
                                 (W == 0 || R.max_pos - K.min_pos < W) && (R.hi - R.lo) == SPINF_SUB && (K.hi - K.lo) == SPINF_SUB) {
                            any = true; all = true;
                        } else {
                            any = false; all = (R.hi - R.lo) == SPINF_SUB && (K.hi - K.lo) == SPINF_SUB;
                            for (int64_t q = R.lo; q < R.hi; q++)
                                for (int64_t k = K.lo; k < K.hi; k++) {
                                    const bool v = visible(art, end, pos, nullptr, 0, W, q, k);
                                    any |= v; all &= v;
                                }
                        }
                        if (any) {
                            bits |= 1u << (2 * w + s);
                            p->active++;
                            if (!all) { bits |= 1u << (8 + 2 * w + s); p->masked++; }
                        }
                    }
                }
                if (bits) {
                    p->kv_idx.push_back((int32_t)j);
                    p->kv_bits.push_back(bits);
                    // the four row groups of a query tile go through its key tiles in step: a key tile costs what its busiest
                    // row group costs, whether the other three have work or not
                    int most = 0;
                    for (int w = 0; w < SPINF_QTILE / SPINF_SUB; w++) most = std::max(most, __builtin_popcount((bits >> (2 * w)) & 3u));
                    weight[t] += (SPINF_QTILE / SPINF_SUB) * most;
                }
            }
            p->qt_ptr[t + 1] = (int32_t)p->kv_idx.size();
        }
        // launch order: runs of query tiles of one job stay together (they share keys), heaviest first inside a run
        p->order.resize(nqt);
        for (int64_t t = 0; t < nqt; t++) p->order[t] = (int32_t)t;
        int64_t a = 0;
        while (a < nqt) {
            int64_t b = a + 1;
            while (b < nqt && group[b] == group[a]) b++;
            std::stable_sort(p->order.begin() + a, p->order.begin() + b, [&](int32_t x, int32_t y) { return weight[x] > weight[y]; });
            a = b;
        }
    } catch (const std::bad_alloc&) {
        delete p;
        return spinf_fail(SPINF_E_NOMEM, "tileplan_build: out of memory");
    }
    *out = p;
    return SPINF_OK;
}

extern "C" int spinf_tileplan_counts(const spinf_tileplan* p, int64_t counts[5]) {
    if (!p || !counts) return spinf_fail(SPINF_E_ARG, "tileplan_counts: null argument");
    counts[0] = (int64_t)p->order.size();
    counts[1] = (int64_t)p->kv_idx.size();
    counts[2] = p->active;
    counts[3] = p->masked;
    counts[4] = p->n;
    return SPINF_OK;
}

extern "C" int spinf_tileplan_export(const spinf_tileplan* p, int32_t* qt_ptr, int32_t* kv_idx, uint32_t* kv_bits, int32_t* order) {
    if (!p || !qt_ptr) return spinf_fail(SPINF_E_ARG, "tileplan_export: null argument");
    if ((!kv_idx || !kv_bits) && !p->kv_idx.empty()) return spinf_fail(SPINF_E_ARG, "tileplan_export: null entry arrays");
    if (!order && !p->order.empty()) return spinf_fail(SPINF_E_ARG, "tileplan_export: null order array");
    std::memcpy(qt_ptr, p->qt_ptr.data(), p->qt_ptr.size() * sizeof(int32_t));
    if (!p->kv_idx.empty()) {
        std::memcpy(kv_idx, p->kv_idx.data(), p->kv_idx.size() * sizeof(int32_t));
        std::memcpy(kv_bits, p->kv_bits.data(), p->kv_bits.size() * sizeof(uint32_t));
    }
    if (!p->order.empty()) std::memcpy(order, p->order.data(), p->order.size() * sizeof(int32_t));
    return SPINF_OK;
}

extern "C" int spinf_tileplan_schedule(const spinf_tileplan* p, int32_t head_groups, int32_t* items, int32_t* list_ptr) {
    if (!p || !list_ptr) return spinf_fail(SPINF_E_ARG, "tileplan_schedule: null argument");
    if (head_groups <= 0 || head_groups >= 4096) return spinf_fail(SPINF_E_ARG, "tileplan_schedule: head groups %d out of range", head_groups);
    const int64_t nqt = (int64_t)p->order.size();
    if (nqt && !items) return spinf_fail(SPINF_E_ARG, "tileplan_schedule: null items");
    if (nqt * head_groups > (int64_t)1 << 30) return spinf_fail(SPINF_E_ARG, "tileplan_schedule: too many items");
    try {
        // items: job run by job run (tiles that share keys), head group by head group, heaviest tile first
        std::vector<int64_t> cum;
        cum.reserve(nqt * head_groups + 1);
        cum.push_back(0);
        int64_t k = 0;
        int64_t a = 0;
        while (a < nqt) {
            int64_t b = a + 1;
            while (b < nqt && p->group[p->order[b]] == p->group[p->order[a]]) b++;
            for (int32_t hp = 0; hp < head_groups; hp++)
                for (int64_t pos = a; pos < b; pos++) {
                    const int32_t t = p->order[pos];
                    const int32_t e0 = p->qt_ptr[t], ne = p->qt_ptr[t + 1] - e0;
                    items[4 * k + 0] = t;
                    items[4 * k + 1] = e0;
                    items[4 * k + 2] = (ne & 0xfffff) | (hp << 20);
                    items[4 * k + 3] = ne > 0 ? p->kv_idx[e0] : 0;
                    cum.push_back(cum.back() + p->weight[t] + 15);   // + a fixed cost per item (queries, output rows; measured ~15 blocks)
                    k++;
                }
            a = b;
        }
        // eight contiguous lists of about equal weight
        const int64_t total = cum.back();
        list_ptr[0] = 0;
        for (int l = 1; l < 8; l++) {
            const int64_t want = total * l / 8;
            const int64_t at = std::lower_bound(cum.begin(), cum.end(), want) - cum.begin();
            list_ptr[l] = (int32_t)std::max<int64_t>(list_ptr[l - 1], std::min<int64_t>(at, k));
        }
        list_ptr[8] = (int32_t)k;
        // The end of a list decides how evenly the workgroups finish: the pass ends up to an item's duration after the lists
        // run dry.  The lightest items of each list (at most TAIL_SHARE of its weight and TAIL_ITEMS items) are therefore
        // moved to its end, heaviest of them first.  A small share on purpose: moved items no longer run next to the items
        // that share their keys (measured on the 24-content pass: 8 % of the weight -1 %, 25 % +2 %, 35 % +3 % kernel time).
        constexpr double TAIL_SHARE = 0.08;
        constexpr int64_t TAIL_ITEMS = 128;
        std::vector<int32_t> idx, moved;
        std::vector<int32_t> tmp;
        for (int l = 0; l < 8; l++) {
            const int64_t lo = list_ptr[l], hi = list_ptr[l + 1];
            if (hi - lo < 3) continue;
            auto cost = [&](int64_t i) { return cum[i + 1] - cum[i]; };
            idx.resize(hi - lo);
            for (int64_t i = lo; i < hi; i++) idx[i - lo] = (int32_t)i;
            std::stable_sort(idx.begin(), idx.end(), [&](int32_t x, int32_t y) { return cost(x) < cost(y); });
            const int64_t budget = (int64_t)(TAIL_SHARE * (double)(cum[hi] - cum[lo]));
            int64_t taken = 0, n_tail = 0;
            while (n_tail < (int64_t)idx.size() && n_tail < TAIL_ITEMS && taken + cost(idx[n_tail]) <= budget) taken += cost(idx[n_tail++]);
            if (n_tail == 0) continue;
            moved.assign((size_t)(hi - lo), 0);
            for (int64_t j = 0; j < n_tail; j++) moved[idx[j] - lo] = 1;
            tmp.clear();
            for (int64_t i = lo; i < hi; i++)
                if (!moved[i - lo]) tmp.insert(tmp.end(), items + 4 * i, items + 4 * i + 4);
            for (int64_t j = n_tail - 1; j >= 0; j--) tmp.insert(tmp.end(), items + 4 * (int64_t)idx[j], items + 4 * (int64_t)idx[j] + 4);
            std::memcpy(items + 4 * lo, tmp.data(), tmp.size() * sizeof(int32_t));
        }
    } catch (const std::bad_alloc&) {
        return spinf_fail(SPINF_E_NOMEM, "tileplan_schedule: out of memory");
    }
    return SPINF_OK;
}

// Static schedule for the kernel with decoupled waves: the items of spinf_tileplan_schedule (same order, same eight lists, one per
// XCD), dealt out to n_lists workgroups by simulating "the workgroup that is free first takes the next item of its XCD's list"
// with a cost model, so that a workgroup's items are known before the launch.  Workgroup b serves list b % 8.  The model is a
// fit to per-workgroup cycle counts of that kernel on the 24-content pass (residual 1.2 %): a workgroup moves through its key
// tiles at about the same pace whatever the number of 32 x 32 blocks its waves compute in them, so an item costs its number of
// key tiles, 0.3 per block that needs the per-element mask (of the busier SIMD pair: SIMDs 0 and 3 run the row groups 0 and 3 of
// a query tile, SIMDs 1 and 2 the row groups 1 and 2) and 3.2 on top (queries, output rows).
extern "C" int spinf_tileplan_schedule_static(const spinf_tileplan* p, int32_t head_groups, int32_t n_lists, int32_t* items, int32_t* list_ptr) {
    if (!p || !list_ptr) return spinf_fail(SPINF_E_ARG, "tileplan_schedule_static: null argument");
    if (n_lists <= 0 || n_lists > 65536) return spinf_fail(SPINF_E_ARG, "tileplan_schedule_static: %d lists out of range", n_lists);
    const int64_t nqt = (int64_t)p->order.size();
    try {
        std::vector<int32_t> base((size_t)std::max<int64_t>(1, nqt * head_groups) * 4);
        int32_t lp[9];
        if (int rc = spinf_tileplan_schedule(p, head_groups, base.data(), lp)) return rc;
        const int nsub = p->ktile / SPINF_SUB;
        std::vector<float> cost(nqt, 0.f);
        for (int64_t t = 0; t < nqt; t++) {
            float tiles = 0.f, ma = 0.f, mb = 0.f;
            for (int32_t e = p->qt_ptr[t]; e < p->qt_ptr[t + 1]; e++) {
                const uint32_t bits = p->kv_bits[e];
                for (int sb = 0; sb < nsub; sb++) {
                    bool any = false;
                    for (int w = 0; w < 4; w++) {
                        if (!((bits >> (2 * w + sb)) & 1u)) continue;
                        any = true;
                        if ((bits >> (8 + 2 * w + sb)) & 1u) (w == 0 || w == 3 ? ma : mb) += 1.f;
                    }
                    if (any) tiles += 1.f;
                }
            }
            // 64-key entries: the lockstep kernels, whose items cost what spinf_tileplan_schedule weighs them with
            cost[t] = p->ktile == SPINF_SUB ? 3.2f + tiles + 0.3f * std::max(ma, mb) : (float)(p->weight[t] + 15);
        }
        const int nl = std::min<int32_t>(8, n_lists);
        std::vector<std::vector<int32_t>> mine((size_t)n_lists);
        std::vector<float> load((size_t)n_lists, 0.f);
        for (int l = 0; l < 8; l++)
            for (int64_t i = lp[l]; i < lp[l + 1]; i++) {
                int best = -1;
                for (int w = l % nl; w < n_lists; w += nl)
                    if (best < 0 || load[w] < load[best]) best = w;
                mine[best].push_back((int32_t)i);
                load[best] += cost[base[4 * i]];
            }
        int64_t k = 0;
        for (int w = 0; w < n_lists; w++) {
            list_ptr[w] = (int32_t)k;
            for (int32_t i : mine[w]) {
                std::memcpy(items + 4 * k, base.data() + 4 * (int64_t)i, 4 * sizeof(int32_t));
                k++;
            }
        }
        list_ptr[n_lists] = (int32_t)k;
    } catch (const std::bad_alloc&) {
        return spinf_fail(SPINF_E_NOMEM, "tileplan_schedule_static: out of memory");
    }
    return SPINF_OK;
}

extern "C" int spinf_tileplan_row0(const spinf_tileplan* p, const int32_t* row_of, int32_t* kv_row0) {
    if (!p || !row_of) return spinf_fail(SPINF_E_ARG, "tileplan_row0: null argument");
    if (!kv_row0 && !p->kv_idx.empty()) return spinf_fail(SPINF_E_ARG, "tileplan_row0: null kv_row0");
    for (size_t e = 0; e < p->kv_idx.size(); e++) {
        const int64_t k0 = (int64_t)p->kv_idx[e] * p->ktile;
        int32_t r0 = k0 + p->ktile <= p->n ? row_of[k0] : -1;
        for (int64_t j = 1; r0 >= 0 && j < p->ktile; j++)
            if (row_of[k0 + j] != r0 + j) r0 = -1;
        kv_row0[e] = r0;
    }
    return SPINF_OK;
}

extern "C" void spinf_tileplan_free(spinf_tileplan* p) { delete p; }
