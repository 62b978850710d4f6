// Plan compiler of the recurrent (Gated DeltaNet) layers: the packed token forest -> segments, levels and kernel calls.
// Stands in for tree_plan (spinf_serve/models/qwen35/qwen.py:158-276); its output is what gdn_tree / gdn_indexed
// (qwen.py:514-590) walk.  Host code, no global state, deterministic.
//
// What it computes.  A token's `prev` is the token before it on its root-to-leaf path.  A *segment* is a maximal run of
// stream-consecutive real tokens that one scan can take in one go: it begins at a real token whose predecessor is missing, is
// not the stream token right before it, or has several children.  Segments form a forest (a segment's parent is the segment of
// its first token's predecessor); the scan of a segment starts from its parent's final state, so segments are run level by level
// and only segments that somebody continues from (or that the caller asks for) leave their state, in a slot of their level.
//
// How.  One pass over the stream numbers the segments and, because a parent always precedes its children in the stream, gives
// their depth at once; a counting sort by depth keeps stream order inside a level; calls are cut from the sorted array.
#include "spinf_tree.h"
#include "common.h"

#include <algorithm>
#include <cstring>
#include <new>
#include <vector>

struct spinf_gdn_plan {
    int64_t n_segments = 0, conv_rows = 0;
    std::vector<int64_t> level_ptr;      // calls of level d: level_ptr[d] .. level_ptr[d+1]
    std::vector<int32_t> call_kind;      // 1 chunked, 0 recurrent
    std::vector<int32_t> call_keep;      // some segment of the call leaves its state
    std::vector<int64_t> call_seg_ptr;   // segments of call c: call_seg_ptr[c] .. call_seg_ptr[c+1] in cu / h0 / ht
    std::vector<int64_t> call_row_ptr;   // rows of call c in idx
    std::vector<int64_t> len, h0, ht;    // per call segment: length, slot of the start state in the level above (-1 zero), slot of its own (-1 none)
    std::vector<int64_t> idx;            // rows of the calls' segments, back to back
    std::vector<int64_t> n_keep;         // slots per level
    std::vector<int64_t> conv;           // [conv_rows, 4]
    std::vector<int64_t> seg_of_row, seg_level, seg_slot;
};

namespace {

struct Seg {
    int64_t first, len, parent;
    int32_t depth;
    bool keeps;
};

}  // namespace

extern "C" int spinf_gdn_plan_build(const int64_t* prev, const uint8_t* real, int64_t n, int32_t path, int32_t short_len, int64_t call_tokens,
                                    int32_t max_init, int64_t rows, const int64_t* keep, int64_t n_keep, spinf_gdn_plan** out) {
    if (!out) return spinf_fail(SPINF_E_ARG, "gdn_plan_build: out is null");
    *out = nullptr;
    if (n < 0 || (n > 0 && (!prev || !real))) return spinf_fail(SPINF_E_ARG, "gdn_plan_build: null stream arrays");
    if (path != 0 && path != 1) return spinf_fail(SPINF_E_ARG, "gdn_plan_build: unknown path %d (0 indexed, 1 levels)", path);
    if (n_keep < 0 || (n_keep > 0 && !keep)) return spinf_fail(SPINF_E_ARG, "gdn_plan_build: null keep list");
    if (path == 1 && max_init <= 0) return spinf_fail(SPINF_E_ARG, "gdn_plan_build: max_init must be positive");
    for (int64_t i = 0; i < n; i++)
        if (prev[i] >= i || prev[i] < -1) return spinf_fail(SPINF_E_ARG, "gdn_plan_build: prev[%lld] = %lld does not point backwards", (long long)i, (long long)prev[i]);
    spinf_gdn_plan* p = new (std::nothrow) spinf_gdn_plan;
    if (!p) return spinf_fail(SPINF_E_NOMEM, "gdn_plan_build: out of memory");
    try {
        // ---- compact rows: real tokens first, in stream order; `rows` doubles as the "no row" value
        int64_t n_real = 0;
        for (int64_t i = 0; i < n; i++) n_real += real[i] != 0;
        const bool compact = rows >= 0;
        if (compact && n_real > rows) {
            delete p;
            return spinf_fail(SPINF_E_ARG, "gdn_plan_build: %lld real tokens do not fit %lld compact rows", (long long)n_real, (long long)rows);
        }
        std::vector<int64_t> row_of;   // stream position -> row of the tensors
        if (compact) {
            row_of.assign(n, rows);
            int64_t r = 0;
            for (int64_t i = 0; i < n; i++)
                if (real[i]) row_of[i] = r++;
        }
        auto row = [&](int64_t i) { return compact ? row_of[i] : i; };

        // ---- segments, in one pass
        std::vector<int32_t> kids(n, 0);
        for (int64_t i = 0; i < n; i++)
            if (prev[i] >= 0) kids[prev[i]]++;
        std::vector<Seg> seg;
        std::vector<int64_t> seg_at(n, -1);
        for (int64_t i = 0; i < n; i++) {
            if (!real[i]) continue;
            const int64_t b = prev[i];
            const bool opens = b < 0 || b != i - 1 || kids[b] > 1;
            if (opens) {
                Seg s;
                s.first = i;
                s.len = 0;
                s.parent = b >= 0 ? seg_at[b] : -1;
                s.depth = s.parent >= 0 ? seg[s.parent].depth + 1 : 0;
                s.keeps = false;
                if (s.parent >= 0) seg[s.parent].keeps = true;   // somebody continues from it
                seg.push_back(s);
            }
            seg_at[i] = (int64_t)seg.size() - 1;
            seg.back().len++;
        }
        for (int64_t j = 0; j < n_keep; j++) {
            const int64_t i = keep[j];
            if (i >= 0 && i < n && real[i]) seg[seg_at[i]].keeps = true;   // the caller wants this segment's state
        }
        const int64_t ns = (int64_t)seg.size();
        p->n_segments = ns;

        // ---- counting sort by depth (stream order inside a level)
        int32_t n_levels = 0;
        for (const Seg& s : seg) n_levels = std::max(n_levels, s.depth + 1);
        std::vector<int64_t> at(n_levels + 1, 0);
        for (const Seg& s : seg) at[s.depth + 1]++;
        for (int32_t d = 0; d < n_levels; d++) at[d + 1] += at[d];
        std::vector<int64_t> by_level(ns);
        {
            std::vector<int64_t> fill(at.begin(), at.end() - 1);
            for (int64_t s = 0; s < ns; s++) by_level[fill[seg[s].depth]++] = s;
        }

        // ---- levels and calls
        p->seg_slot.assign(ns, -1);
        p->seg_level.resize(ns);
        for (int64_t s = 0; s < ns; s++) p->seg_level[s] = seg[s].depth;
        p->level_ptr.push_back(0);
        p->call_seg_ptr.push_back(0);
        p->call_row_ptr.push_back(0);
        auto emit = [&](const int64_t* first, const int64_t* last, int32_t kind, int32_t level) {   // one call over these segments
            bool any_keep = false;
            for (const int64_t* it = first; it != last; ++it) {
                const Seg& s = seg[*it];
                p->len.push_back(s.len);
                p->h0.push_back(level > 0 && s.parent >= 0 ? p->seg_slot[s.parent] : -1);
                p->ht.push_back(s.keeps ? p->seg_slot[*it] : -1);
                any_keep |= s.keeps;
                for (int64_t t = 0; t < s.len; t++) p->idx.push_back(row(s.first + t));
            }
            p->call_kind.push_back(kind);
            p->call_keep.push_back(any_keep);
            p->call_seg_ptr.push_back((int64_t)p->len.size());
            p->call_row_ptr.push_back((int64_t)p->idx.size());
        };
        std::vector<int64_t> group;
        for (int32_t d = 0; d < n_levels; d++) {
            const int64_t* lo = by_level.data() + at[d];
            const int64_t* hi = by_level.data() + at[d + 1];
            if (path == 0) {
                // slots of the level: its keeping segments, in stream order
                int64_t slots = 0;
                for (const int64_t* it = lo; it != hi; ++it)
                    if (seg[*it].keeps) p->seg_slot[*it] = slots++;
                p->n_keep.push_back(slots);
                // the long segments go to the chunked kernel, cut into calls of at most call_tokens tokens (a call holds at
                // least one segment); the short ones to the recurrent kernel in one call
                for (int32_t kind = 1; kind >= 0; kind--) {
                    group.clear();
                    for (const int64_t* it = lo; it != hi; ++it)
                        if ((seg[*it].len > short_len) == (kind == 1)) group.push_back(*it);
                    if (group.empty()) continue;
                    int64_t total = 0;
                    for (int64_t g : group) total += seg[g].len;
                    size_t a = 0;
                    while (a < group.size()) {
                        size_t b = group.size();
                        if (kind == 1 && total > call_tokens) {
                            int64_t tokens = seg[group[a]].len;
                            b = a + 1;
                            while (b < group.size() && tokens + seg[group[b]].len <= call_tokens) tokens += seg[group[b++]].len;
                        }
                        emit(group.data() + a, group.data() + b, kind, d);
                        a = b;
                    }
                }
            } else {
                // levels path: the segments that keep their state first (their slots number them), then the others; below the
                // roots a call takes at most max_init segments (each starts from a copy of its parent's state)
                int64_t slots = 0;
                for (int pass = 0; pass < 2; pass++) {
                    group.clear();
                    for (const int64_t* it = lo; it != hi; ++it)
                        if (seg[*it].keeps == (pass == 0)) group.push_back(*it);
                    if (group.empty()) continue;
                    if (pass == 0)
                        for (int64_t g : group) p->seg_slot[g] = slots++;
                    const size_t step = d == 0 ? group.size() : (size_t)max_init;
                    for (size_t a = 0; a < group.size(); a += step) {
                        const size_t b = std::min(group.size(), a + step);
                        int64_t longest = 0;
                        for (size_t g = a; g < b; g++) longest = std::max(longest, seg[group[g]].len);
                        emit(group.data() + a, group.data() + b, longest > 64 ? 1 : 0, d);
                        p->call_keep.back() = pass == 0;
                    }
                }
                p->n_keep.push_back(slots);
            }
            p->level_ptr.push_back((int64_t)p->call_kind.size());
        }

        // ---- convolution taps: the three tokens before a token on its path, oldest first, then the token itself
        const int64_t none = compact ? rows : n;
        p->conv_rows = compact ? rows : n;
        p->conv.assign((size_t)p->conv_rows * 4, none);
        for (int64_t i = 0; i < n; i++) {
            if (compact && !real[i]) continue;
            int64_t* tap = p->conv.data() + 4 * row(i);
            tap[3] = row(i);
            int64_t hop = real[i] ? prev[i] : -1;
            for (int back = 2; back >= 0 && hop >= 0; back--) {
                tap[back] = row(hop);
                hop = prev[hop];
            }
        }
        p->seg_of_row.assign((size_t)p->conv_rows, -1);
        for (int64_t i = 0; i < n; i++)
            if (real[i]) p->seg_of_row[row(i)] = seg_at[i];
    } catch (const std::bad_alloc&) {
        delete p;
        return spinf_fail(SPINF_E_NOMEM, "gdn_plan_build: out of memory");
    }
    *out = p;
    return SPINF_OK;
}

extern "C" int spinf_gdn_plan_counts(const spinf_gdn_plan* p, int64_t counts[6]) {
    if (!p || !counts) return spinf_fail(SPINF_E_ARG, "gdn_plan_counts: null argument");
    counts[0] = p->n_segments;
    counts[1] = (int64_t)p->level_ptr.size() - 1;
    counts[2] = (int64_t)p->call_kind.size();
    counts[3] = (int64_t)p->len.size();
    counts[4] = (int64_t)p->idx.size();
    counts[5] = p->conv_rows;
    return SPINF_OK;
}

extern "C" int spinf_gdn_plan_export(const spinf_gdn_plan* p, int64_t* level_ptr, int32_t* call_kind, int32_t* call_keep, int64_t* call_seg_ptr,
                                     int64_t* call_row_ptr, int64_t* seg_len, int64_t* h0_idx, int64_t* ht_idx, int64_t* idx, int64_t* n_keep,
                                     int64_t* conv, int64_t* seg_of_row, int64_t* seg_level, int64_t* seg_slot) {
    if (!p || !level_ptr || !call_seg_ptr || !call_row_ptr) return spinf_fail(SPINF_E_ARG, "gdn_plan_export: null argument");
    auto put = [](auto* dst, const auto& src) -> bool {
        if (src.empty()) return true;
        if (!dst) return false;
        std::memcpy(dst, src.data(), src.size() * sizeof(src[0]));
        return true;
    };
    const bool ok = put(level_ptr, p->level_ptr) && put(call_kind, p->call_kind) && put(call_keep, p->call_keep) && put(call_seg_ptr, p->call_seg_ptr) &&
                    put(call_row_ptr, p->call_row_ptr) && put(seg_len, p->len) && put(h0_idx, p->h0) && put(ht_idx, p->ht) && put(idx, p->idx) &&
                    put(n_keep, p->n_keep) && put(conv, p->conv) && put(seg_of_row, p->seg_of_row) && put(seg_level, p->seg_level) && put(seg_slot, p->seg_slot);
    if (!ok) return spinf_fail(SPINF_E_ARG, "gdn_plan_export: null array for a non-empty part of the plan");
    return SPINF_OK;
}

extern "C" void spinf_gdn_plan_free(spinf_gdn_plan* p) { delete p; }
