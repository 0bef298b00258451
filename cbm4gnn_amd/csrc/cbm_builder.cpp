// Host-side construction of the CBM (compressed binary matrix) format.
//
// Replaces the reference builders cbm_init_v1_/_v2_ (/root/reference/cbm/cbm_extensions.cpp:8-326,
// :328-644).  Same mathematics -- distance graph with the alpha admission rule (:75-103), a
// minimum spanning arborescence rooted at a virtual node (the reference calls arbok::TarjanPQ,
// :109-148), signed row deltas by a sorted merge (:186-261) -- but a different product: instead
// of a delta COO with fp32 values and a tree CSR only, it emits the device format the HIP kernels
// consume:
//   rowptr[N+1]      CSR offsets of the delta matrix
//   idx[nnz]         column | (negative ? 1u<<31 : 0), columns ascending within a row
//   parent[N]        parent row, -1 for children of the virtual root
//   order[N]         rows sorted by (tree level, id); level 0 = children of the root
//   level_off[L+1]   offsets of the levels inside order[]
// plus the reference's own tree arrays mst_row[N+2] / mst_col[N] (:274-286) so that code written
// against the reference's cbm_matrix attributes keeps working.
//
// Differences in method (none in result class):
//   * |row_i ^ row_j| is streamed row by row with a sparse accumulator and only admissible pairs
//     are kept; the reference materialises all of A*A^T with mkl_sparse_syrk (:46-65).
//   * the arborescence is found by an own implementation of Tarjan's O(m log n) algorithm
//     (sorted runs merged through small heaps, lazy reduced costs, union-find with rollback
//     for the expansion).
//   * the normalisation vector is NOT folded into delta values here; kernels apply it.
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <new>
#include <utility>
#include <vector>
#include <omp.h>

#include "../../include/cbm_hip.h"

namespace {

struct CandEdge { int32_t u, v, w; };

// Stable parallel bucketing (a counting sort): item t of `count` goes to bucket key(t) in
// [0, n_buckets); offsets[] (n_buckets + 1) is computed, place(t, position) stores the item.
// Items keep their order inside a bucket: the threads take consecutive chunks of the items and
// count their chunk per bucket; a prefix over (bucket, chunk) gives every chunk its own range.
// Fewer chunks than threads when threads x buckets counters would be too many; one for small inputs.
template <class Key, class Place>
void bucket_stable(int64_t count, int32_t n_buckets, std::vector<int64_t>& offsets, int threads, Key key, Place place) {
    // at most 2^26 counters (512 MB) in all
    int chunks = (int)std::max<int64_t>(1, std::min<int64_t>(threads, ((int64_t)1 << 26) / std::max(n_buckets, 1)));
    if (count < (int64_t)1 << 16) chunks = 1;
    std::vector<int64_t> start((size_t)chunks * n_buckets);
    const int64_t per = (count + chunks - 1) / chunks;
#pragma omp parallel for schedule(static, 1) num_threads(chunks)
    for (int c = 0; c < chunks; c++) {
        int64_t* mine = start.data() + (size_t)c * n_buckets;
        std::fill(mine, mine + n_buckets, 0);
        const int64_t lo = std::min(count, c * per), hi = std::min(count, lo + per);
        for (int64_t t = lo; t < hi; t++) mine[key(t)]++;
    }
    offsets.assign((size_t)n_buckets + 1, 0);
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int32_t b = 0; b < n_buckets; b++) {
        int64_t size = 0;
        for (int c = 0; c < chunks; c++) size += start[(size_t)c * n_buckets + b];
        offsets[b + 1] = size;
    }
    for (int32_t b = 0; b < n_buckets; b++) offsets[b + 1] += offsets[b];
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int32_t b = 0; b < n_buckets; b++) {
        int64_t at = offsets[b];
        for (int c = 0; c < chunks; c++) {
            int64_t& slot = start[(size_t)c * n_buckets + b];
            const int64_t size = slot;
            slot = at;
            at += size;
        }
    }
#pragma omp parallel for schedule(static, 1) num_threads(chunks)
    for (int c = 0; c < chunks; c++) {
        int64_t* mine = start.data() + (size_t)c * n_buckets;
        const int64_t lo = std::min(count, c * per), hi = std::min(count, lo + per);
        for (int64_t t = lo; t < hi; t++) place(t, mine[key(t)]++);
    }
}

// ---------------------------------------------------------------------------------------------
// Minimum spanning arborescence (Tarjan 1977 / Camerini-Fratta-Maffioli 1979 expansion).
//
// The edges entering a (contracted) node are kept as a k-way merge instead of a meldable heap:
// every original node's incoming edges form one run, sorted once by (weight, edge id); a
// contracted node owns the runs of its members and a small binary heap over the runs' current
// heads.  Popping the cheapest entering edge advances one run (sequential memory) and sifts
// one entry of a heap that fits the L1 cache; contracting a cycle moves the smaller heaps
// into the largest.  Reduced costs are lazy: an offset per contracted node plus an offset per
// run that absorbs the difference when the run changes owner.  Ties go to the smaller edge id,
// so the result does not depend on the order in which heaps were merged.
// ---------------------------------------------------------------------------------------------
class Arborescence {
public:
    Arborescence(int32_t n, const std::vector<CandEdge>& edges, int threads)
        : n_(n), threads_(threads), edges_(edges), uf_(n, -1), fast_(n) {}

    // Returns total weight; par[v] = tail of the edge entering v (par[root] = -1).
    int64_t run(int32_t root, std::vector<int32_t>& par) {
        const int64_t m = (int64_t)edges_.size();
        // runs: edges grouped by head, each group sorted by (weight, id); weight and tail are
        // copied next to the id so that walking a run never touches edges_
        run_id_.resize(m); run_w_.resize(m); run_tail_.resize(m);
        bucket_stable(m, n_, run_beg_, threads_, [&](int64_t e) { return edges_[e].v; },
                      [&](int64_t e, int64_t at) { run_id_[at] = (int32_t)e; });
#pragma omp parallel for schedule(dynamic, 64) num_threads(threads_)
        for (int32_t v = 0; v < n_; v++) {
            const int64_t b = run_beg_[v], e = run_beg_[v + 1];
            std::sort(run_id_.begin() + b, run_id_.begin() + e, [&](int32_t x, int32_t y) {
                return edges_[x].w != edges_[y].w ? edges_[x].w < edges_[y].w : x < y;
            });
            for (int64_t k = b; k < e; k++) { run_w_[k] = edges_[run_id_[k]].w; run_tail_[k] = edges_[run_id_[k]].u; }
        }
        pos_.assign(run_beg_.begin(), run_beg_.end() - 1);
        run_off_.assign(n_, 0);
        queue_.assign(n_, {});
        queue_of_.resize(n_);
        queue_off_.assign(n_, 0);
        for (int32_t v = 0; v < n_; v++) {
            fast_[v] = v;
            queue_of_[v] = v;
            if (run_beg_[v] < run_beg_[v + 1]) queue_[v].push_back({(int64_t)run_w_[run_beg_[v]], run_id_[run_beg_[v]], v});
        }

        std::vector<int32_t> seen(n_, -1), path(n_), Q(n_), in(n_, -1), members;
        seen[root] = root;
        int64_t res = 0;
        struct Cycle { int32_t node; int32_t time; int32_t eb, ee; };
        std::vector<Cycle> cycles;
        std::vector<int32_t> cyc_edges;
        for (int32_t s = 0; s < n_; s++) {
            int32_t u = s, qi = 0;
            while (seen[u] < 0) {
                const int32_t q = queue_of_[u];
                std::vector<Head>& heap = queue_[q];
                if (heap.empty()) return -1;             // node not reachable from the root
                const Head top = heap[0];
                const int32_t e = top.id;
                const int64_t w = top.key + queue_off_[q];            // reduced cost of e
                const int32_t tail = run_tail_[pos_[top.run]];
                advance(heap, top.run, u);                             // pop
                // An edge inside the (contracted) node is dropped outright.  Charging its reduced
                // cost and discounting the rest of the queue by it, as for any other popped edge,
                // would cancel out with the next pop, and the one-edge "cycle" it would record
                // expands to nothing.
                if (find_fast(tail) == u) continue;
                queue_off_[q] -= w;                                    // remaining keys become reduced costs
                Q[qi] = e; path[qi++] = u; seen[u] = s;
                res += w;
                u = find_fast(tail);
                if (seen[u] == s) {                      // closed a cycle: contract it into u
                    const int32_t end = qi, time = (int32_t)hist_.size();
                    members.clear();
                    int32_t x;
                    do { x = path[--qi]; members.push_back(queue_of_[x]); } while (join(u, x));
                    u = find_fast(u);
                    queue_of_[u] = merge_queues(members);
                    seen[u] = -1;
                    cycles.push_back({u, time, (int32_t)cyc_edges.size(), (int32_t)cyc_edges.size() + (end - qi)});
                    for (int32_t i = qi; i < end; i++) cyc_edges.push_back(Q[i]);
                }
            }
            for (int32_t i = 0; i < qi; i++) in[find(edges_[Q[i]].v)] = Q[i];
        }
        for (int64_t c = (int64_t)cycles.size() - 1; c >= 0; c--) {   // expand, most recent first
            const Cycle& cy = cycles[c];
            rollback(cy.time);
            const int32_t in_edge = in[cy.node];
            for (int32_t i = cy.eb; i < cy.ee; i++) in[find(edges_[cyc_edges[i]].v)] = cyc_edges[i];
            in[find(edges_[in_edge].v)] = in_edge;
        }
        par.assign(n_, -1);
        for (int32_t v = 0; v < n_; v++) if (v != root) par[v] = edges_[in[v]].u;
        return res;
    }

private:
    struct Head { int64_t key; int32_t id, run; };              // head of a run; key excludes the owner's offset
    static bool before(const Head& a, const Head& b) { return a.key != b.key ? a.key < b.key : a.id < b.id; }

    int32_t n_;
    int threads_;
    const std::vector<CandEdge>& edges_;
    std::vector<int64_t> run_beg_, pos_;                        // per original node: its run and the next unread entry
    std::vector<int32_t> run_id_, run_w_, run_tail_;            // per run entry: edge id, weight, tail
    std::vector<int64_t> run_off_;                              // per run: offset relative to its owner's
    std::vector<std::vector<Head>> queue_;                      // binary min-heaps over run heads
    std::vector<int32_t> queue_of_;                             // per representative: index of its queue
    std::vector<int64_t> queue_off_;                            // per queue: offset of every key in it
    std::vector<int32_t> uf_;                                   // <0: -size, else parent (no compression: undoable)
    std::vector<int32_t> fast_;                                 // the same sets with path halving, for the forward pass
    std::vector<std::pair<int32_t, int32_t>> hist_;

    static void sift_down(std::vector<Head>& h, size_t i) {
        const size_t n = h.size();
        const Head x = h[i];
        for (;;) {
            size_t c = 2 * i + 1;
            if (c >= n) break;
            if (c + 1 < n && before(h[c + 1], h[c])) c++;
            if (!before(h[c], x)) break;
            h[i] = h[c];
            i = c;
        }
        h[i] = x;
    }
    static void sift_up(std::vector<Head>& h, size_t i) {
        const Head x = h[i];
        while (i > 0) {
            const size_t p = (i - 1) / 2;
            if (!before(x, h[p])) break;
            h[i] = h[p];
            i = p;
        }
        h[i] = x;
    }
    // The run at the top of the heap moves on to its next entry (or leaves the heap).  Entries
    // whose tail already lies inside the owner `u` are skipped on the way: they stay internal
    // for good and would only be dropped when they reached the top.
    void advance(std::vector<Head>& h, int32_t run, int32_t u) {
        const int64_t end = run_beg_[run + 1];
        int64_t k = pos_[run] + 1;
        while (k < end && find_fast(run_tail_[k]) == u) k++;
        pos_[run] = k;
        if (k < end) {
            h[0] = {(int64_t)run_w_[k] + run_off_[run], run_id_[k], run};
        } else {
            h[0] = h.back();
            h.pop_back();
            if (h.empty()) return;
        }
        sift_down(h, 0);
    }
    // All queues in `which` (distinct) become one: the smaller ones are moved into the largest.
    int32_t merge_queues(const std::vector<int32_t>& which) {
        int32_t base = which[0];
        for (int32_t q : which) if (queue_[q].size() > queue_[base].size()) base = q;
        std::vector<Head>& dst = queue_[base];
        const size_t before_size = dst.size();
        for (int32_t q : which) {
            if (q == base) continue;
            const int64_t delta = queue_off_[q] - queue_off_[base];
            for (Head hd : queue_[q]) {
                hd.key += delta;
                run_off_[hd.run] += delta;
                dst.push_back(hd);
            }
            std::vector<Head>().swap(queue_[q]);
        }
        const size_t added = dst.size() - before_size;
        if (added * 8 > dst.size()) {
            for (size_t i = dst.size() / 2; i-- > 0;) sift_down(dst, i);   // rebuild
        } else {
            for (size_t i = before_size; i < dst.size(); i++) sift_up(dst, i);
        }
        return base;
    }
    int32_t find(int32_t x) const { while (uf_[x] >= 0) x = uf_[x]; return x; }
    int32_t find_fast(int32_t x) {
        while (fast_[x] != x) { fast_[x] = fast_[fast_[x]]; x = fast_[x]; }
        return x;
    }
    bool join(int32_t a, int32_t b) {
        a = find(a); b = find(b);
        if (a == b) return false;
        if (uf_[a] > uf_[b]) std::swap(a, b);
        hist_.push_back({a, uf_[a]}); hist_.push_back({b, uf_[b]});
        uf_[a] += uf_[b]; uf_[b] = a;
        fast_[b] = a;                                            // same representative in both structures
        return true;
    }
    void rollback(int32_t t) {
        for (int32_t i = (int32_t)hist_.size(); i-- > t;) uf_[hist_[i].first] = hist_[i].second;
        hist_.resize(t);
    }
};

template <class T> T* dup_array(const std::vector<T>& v) {
    T* p = (T*)std::malloc(sizeof(T) * (v.size() ? v.size() : 1));
    if (!p) throw std::bad_alloc();
    if (!v.empty()) std::memcpy(p, v.data(), sizeof(T) * v.size());
    return p;
}


// The input matrix as the stages of the build see it.
struct Graph {
    int32_t N = 0;
    int64_t nnzA = 0;
    bool symmetric = false;
    std::vector<int64_t> rp, tp;         // CSR offsets of A and of A^T
    std::vector<int32_t> ci, tr;         // columns of A (ascending per row), rows of A^T (ascending per column)
    std::vector<int32_t> nnz;            // entries per row of A
    std::vector<int64_t> after;          // per entry k = (r, c) of A: first position in tr of a row id > r inside column c
};

// COO -> CSR(A) with sorted unique columns, and its transpose.
int build_graph(const int32_t* row, const int32_t* col, int64_t E, int32_t N, int threads, Graph& g) {
    g.N = N;
    std::vector<int64_t>& rp = g.rp; std::vector<int32_t>& ci = g.ci; std::vector<int32_t>& nnz = g.nnz;
    std::vector<int64_t>& tp = g.tp; std::vector<int32_t>& tr = g.tr;
    bool bad = false;
#pragma omp parallel for schedule(static) num_threads(threads) reduction(|| : bad)
    for (int64_t k = 0; k < E; k++) bad = bad || row[k] < 0 || row[k] >= N || col[k] < 0 || col[k] >= N;
    if (bad) return CBM_ERR_SHAPE;
    ci.resize(E);
    bucket_stable(E, N, rp, threads, [&](int64_t k) { return row[k]; }, [&](int64_t k, int64_t at) { ci[at] = col[k]; });
    nnz.resize(N);
#pragma omp parallel for schedule(dynamic, 256) num_threads(threads)
    for (int32_t r = 0; r < N; r++) {
        auto b = ci.begin() + rp[r], e = ci.begin() + rp[r + 1];
        std::sort(b, e);
        nnz[r] = (int32_t)(std::unique(b, e) - b);
    }
    {   // compact duplicates away
        int64_t w = 0;
        for (int32_t r = 0; r < N; r++) {
            const int64_t b = rp[r];
            rp[r] = w;
            if (w != b) std::memmove(&ci[w], &ci[b], sizeof(int32_t) * (size_t)nnz[r]);
            w += nnz[r];
        }
        rp[N] = w;
        ci.resize(w);
    }
    g.nnzA = rp[N];
    // transpose: entry k = (r, c) goes to column c; entries arrive in ascending r, so every column
    // of A^T lists its rows in ascending order and after[k] is the position behind the entry
    std::vector<int32_t> row_of(g.nnzA);
#pragma omp parallel for schedule(dynamic, 256) num_threads(threads)
    for (int32_t r = 0; r < N; r++)
        for (int64_t k = rp[r]; k < rp[r + 1]; k++) row_of[k] = r;
    tr.resize(g.nnzA);
    g.after.resize(g.nnzA);
    bucket_stable(g.nnzA, N, tp, threads, [&](int64_t k) { return ci[k]; },
                  [&](int64_t k, int64_t at) { tr[at] = row_of[k]; g.after[k] = at + 1; });
    // symmetric pattern <=> CSR(A) == CSR(A^T) (both have ascending columns)
    g.symmetric = rp == tp && ci == tr;
    return CBM_OK;
}

// Candidate edges of the distance graph (reference rule, cbm_extensions.cpp:75-103) from the
// admissible pairs of one row i, in the reference's emission order: the edge from the virtual
// root, then for every j > i ascending the edges j -> i and i -> j.
//   pair (i, j>i) with s shared columns: h = nnz_i + nnz_j - 2s;
//   j -> i admitted iff h < nnz_i - alpha  <=>  2s > nnz_j + alpha
//   i -> j admitted iff h < nnz_j - alpha  <=>  2s > nnz_i + alpha
inline void emit_row(const Graph& g, int32_t alpha, int32_t i, std::vector<std::pair<int32_t, int32_t>>& adm,
                     std::vector<CandEdge>& o) {
    const int32_t ni = g.nnz[i];
    o.push_back({g.N, i, ni});
    std::sort(adm.begin(), adm.end());
    for (auto& js : adm) {
        const int32_t j = js.first, nj = g.nnz[j];
        const int32_t h = ni + nj - 2 * js.second;
        if (h < ni - alpha) o.push_back({j, i, h});
        if (h < nj - alpha) o.push_back({i, j, h});
    }
}

inline int concat_chunks(std::vector<std::vector<CandEdge>>& chunk_out, std::vector<CandEdge>& cand) {
    size_t tot = 0;
    for (auto& o : chunk_out) tot += o.size();
    if (tot >= (size_t)INT32_MAX) return CBM_ERR_SHAPE;
    cand.reserve(tot);
    for (auto& o : chunk_out) { cand.insert(cand.end(), o.begin(), o.end()); std::vector<CandEdge>().swap(o); }
    return CBM_OK;
}

// Row intersections on the host: |row_i ^ row_j| streamed row by row with a per-thread sparse
// accumulator, only admissible pairs kept.
int candidates_host(const Graph& g, int32_t alpha, int threads, std::vector<CandEdge>& cand) {
    const int32_t N = g.N;
    const int32_t CH = 64;
    const int32_t n_chunks = (N + CH - 1) / CH;
    std::vector<std::vector<CandEdge>> chunk_out(n_chunks);
#pragma omp parallel num_threads(threads)
    {
        std::vector<int32_t> cnt(N, 0), touched;
        std::vector<std::pair<int32_t, int32_t>> adm;
        touched.reserve(1024);
#pragma omp for schedule(dynamic, 1)
        for (int32_t ch = 0; ch < n_chunks; ch++) {
            std::vector<CandEdge>& o = chunk_out[ch];
            const int32_t i_end = std::min(N, (ch + 1) * CH);
            for (int32_t i = ch * CH; i < i_end; i++) {
                const int32_t ni = g.nnz[i];
                touched.clear();
                for (int64_t k = g.rp[i]; k < g.rp[i + 1]; k++) {
                    const int32_t* q = g.tr.data() + g.after[k];
                    const int32_t* hi = g.tr.data() + g.tp[g.ci[k] + 1];
                    for (; q < hi; ++q) {
                        const int32_t j = *q;
                        if (cnt[j]++ == 0) touched.push_back(j);
                    }
                }
                adm.clear();
                for (int32_t j : touched) {
                    const int32_t s = cnt[j];
                    cnt[j] = 0;
                    if (2 * s > std::min(ni, g.nnz[j]) + alpha) adm.push_back({j, s});
                }
                emit_row(g, alpha, i, adm, o);
            }
        }
    }
    return concat_chunks(chunk_out, cand);
}

// The same candidate list from row intersections computed elsewhere (on the GPU): pairs (i, j, s)
// with i < j and s = |row_i ^ row_j|, in any order, holding at least every admissible pair.
int candidates_from_pairs(const Graph& g, int32_t alpha, const cbm_pair* pairs, int64_t n_pairs, int threads,
                          std::vector<CandEdge>& cand) {
    const int32_t N = g.N;
    bool bad = false;
#pragma omp parallel for schedule(static) num_threads(threads) reduction(|| : bad)
    for (int64_t p = 0; p < n_pairs; p++) {
        const cbm_pair& q = pairs[p];
        bad = bad || q.i < 0 || q.j <= q.i || q.j >= N || q.s <= 0 || q.s > std::min(g.nnz[q.i], g.nnz[q.j]);
    }
    if (bad) return CBM_ERR_SHAPE;
    std::vector<int64_t> first;
    std::vector<std::pair<int32_t, int32_t>> by_row(n_pairs);
    bucket_stable(n_pairs, N, first, threads, [&](int64_t p) { return pairs[p].i; },
                  [&](int64_t p, int64_t at) { by_row[at] = {pairs[p].j, pairs[p].s}; });
    const int32_t CH = 64;
    const int32_t n_chunks = (N + CH - 1) / CH;
    std::vector<std::vector<CandEdge>> chunk_out(n_chunks);
    bool duplicate = false;
#pragma omp parallel num_threads(threads)
    {
        std::vector<std::pair<int32_t, int32_t>> adm;
#pragma omp for schedule(dynamic, 1)
        for (int32_t ch = 0; ch < n_chunks; ch++) {
            const int32_t i_end = std::min(N, (ch + 1) * CH);
            for (int32_t i = ch * CH; i < i_end; i++) {
                adm.clear();
                for (int64_t p = first[i]; p < first[i + 1]; p++)
                    if (2 * by_row[p].second > std::min(g.nnz[i], g.nnz[by_row[p].first]) + alpha) adm.push_back(by_row[p]);
                emit_row(g, alpha, i, adm, chunk_out[ch]);              // sorts adm by j
                for (size_t a = 1; a < adm.size(); a++)
                    if (adm[a].first == adm[a - 1].first) {
#pragma omp atomic write
                        duplicate = true;
                    }
            }
        }
    }
    if (duplicate) return CBM_ERR_SHAPE;
    return concat_chunks(chunk_out, cand);
}

// seconds spent by the last build of this thread in: CSR + transpose, candidate edges,
// arborescence, tree arrays + deltas
thread_local double g_last_timings[4] = {0, 0, 0, 0};

// Arborescence, tree arrays, signed deltas.
int finish_format(const Graph& g, std::vector<CandEdge>& cand, int threads, int32_t max_levels, cbm_format* out,
                  double t_mark) {
    const int32_t N = g.N;
    const std::vector<int64_t>& rp = g.rp; const std::vector<int32_t>& ci = g.ci; const std::vector<int32_t>& nnz = g.nnz;
    const int64_t nnzA = g.nnzA;
    const bool symmetric = g.symmetric;
    auto lap = [&](int slot) { const double t = omp_get_wtime(); g_last_timings[slot] = t - t_mark; t_mark = t; };
    {
        // ---- arborescence ----------------------------------------------------------------------
        std::vector<int32_t> par;
        int64_t weight;
        {
            Arborescence msa(N + 1, cand, threads);
            weight = msa.run(N, par);
        }
        if (weight < 0) return CBM_ERR_INTERNAL;
        const int64_t n_cand = (int64_t)cand.size();
        std::vector<CandEdge>().swap(cand);

        lap(2);
        // ---- tree arrays: children ascending per parent; levels by BFS --------------------------
        std::vector<int32_t> mst_row, mst_col(N);
        auto children_of = [&]() {
            mst_row.assign(N + 2, 0);
            for (int32_t v = 0; v < N; v++) mst_row[par[v] + 1]++;
            for (int32_t u = 0; u <= N; u++) mst_row[u + 1] += mst_row[u];
            std::vector<int32_t> fill(mst_row.begin(), mst_row.end() - 1);
            for (int32_t v = 0; v < N; v++) mst_col[fill[par[v]]++] = v;
        };
        children_of();
        bool cut_any = false;
        if (max_levels > 0) {
            // Depth limit: a row that would land on level max_levels is re-attached to the virtual
            // root (its delta becomes the whole row) and its subtree moves up with it.  Every tree
            // level costs the multiply a dependent launch, so a few extra delta entries can be the
            // better deal; the result is still a valid format, only no longer of minimum weight.
            std::vector<int32_t> lvl(N, 0), queue(N);
            int32_t head = 0, tail = 0;
            for (int32_t q = mst_row[N]; q < mst_row[N + 1]; q++) queue[tail++] = mst_col[q];
            while (head < tail) {
                const int32_t u = queue[head++];
                for (int32_t q = mst_row[u]; q < mst_row[u + 1]; q++) {
                    const int32_t c = mst_col[q];
                    lvl[c] = lvl[u] + 1;
                    if (lvl[c] >= max_levels) { par[c] = N; lvl[c] = 0; cut_any = true; }
                    queue[tail++] = c;
                }
            }
            if (tail != N) return CBM_ERR_INTERNAL;
            if (cut_any) children_of();
        }
        std::vector<int32_t> level(N, -1), order(N), level_off;
        {
            int32_t head = 0, tail = 0;
            for (int32_t q = mst_row[N]; q < mst_row[N + 1]; q++) { level[mst_col[q]] = 0; order[tail++] = mst_col[q]; }
            level_off.push_back(0);
            int32_t cur = 0;
            while (head < tail) {
                const int32_t u = order[head];
                if (level[u] != cur) { level_off.push_back(head); cur = level[u]; }
                head++;
                for (int32_t q = mst_row[u]; q < mst_row[u + 1]; q++) { level[mst_col[q]] = level[u] + 1; order[tail++] = mst_col[q]; }
            }
            if (tail != N) return CBM_ERR_INTERNAL;
            level_off.push_back(N);
            // BFS yields (level, parent-visit) order; the format wants (level, id)
            for (size_t l = 0; l + 1 < level_off.size(); l++)
                std::sort(order.begin() + level_off[l], order.begin() + level_off[l + 1]);
        }

        // ---- signed deltas, packed --------------------------------------------------------------
        std::vector<int32_t> drp(N + 1, 0);
#pragma omp parallel for schedule(dynamic, 256) num_threads(threads)
        for (int32_t v = 0; v < N; v++) {
            const int32_t u = par[v];
            int32_t c = 0;
            if (u == N) c = nnz[v];
            else {
                int64_t a = rp[u], ae = rp[u + 1], b = rp[v], be = rp[v + 1];
                while (a < ae && b < be) {
                    if (ci[a] == ci[b]) { a++; b++; }
                    else if (ci[a] > ci[b]) { c++; b++; }
                    else { c++; a++; }
                }
                c += (int32_t)((ae - a) + (be - b));
            }
            drp[v + 1] = c;
        }
        int64_t run = 0;
        for (int32_t v = 0; v < N; v++) { run += drp[v + 1]; if (run > INT32_MAX) return CBM_ERR_SHAPE; drp[v + 1] = (int32_t)run; }
        if (!cut_any && run != weight) return CBM_ERR_INTERNAL;      // nnz(delta) must equal the arborescence weight
        std::vector<uint32_t> idx(run);
#pragma omp parallel for schedule(dynamic, 256) num_threads(threads)
        for (int32_t v = 0; v < N; v++) {
            const int32_t u = par[v];
            uint32_t* o = idx.data() + drp[v];
            int64_t b = rp[v], be = rp[v + 1];
            if (u == N) { for (; b < be; b++) *o++ = (uint32_t)ci[b]; continue; }
            int64_t a = rp[u], ae = rp[u + 1];
            while (a < ae && b < be) {
                if (ci[a] == ci[b]) { a++; b++; }
                else if (ci[a] > ci[b]) *o++ = (uint32_t)ci[b++];
                else *o++ = (uint32_t)ci[a++] | 0x80000000u;
            }
            for (; a < ae; a++) *o++ = (uint32_t)ci[a] | 0x80000000u;
            for (; b < be; b++) *o++ = (uint32_t)ci[b];
        }
        std::vector<int32_t> parent(N);
        for (int32_t v = 0; v < N; v++) parent[v] = par[v] == N ? -1 : par[v];

        lap(3);
        out->n = N; out->nnz = run; out->n_levels = (int32_t)level_off.size() - 1;
        out->n_candidates = n_cand; out->msa_weight = weight; out->nnz_a = nnzA;
        out->is_symmetric = symmetric ? 1 : 0;
        out->rowptr = dup_array(drp); out->idx = dup_array(idx); out->parent = dup_array(parent);
        out->order = dup_array(order); out->level_off = dup_array(level_off);
        out->mst_row = dup_array(mst_row); out->mst_col = dup_array(mst_col);
        return CBM_OK;
    }
}

}  // namespace

struct cbm_builder {
    Graph g;
    int threads = 1;
    int32_t max_levels = 0;      // 0 = no limit
};

namespace {

// Pieces of row r under a cut plan: the row's entries are cut where the column passes from one
// column block to the next (col_blocks >= 2: blocks of ceil(n / col_blocks) consecutive columns; the
// entries of a row are sorted by column, so a block's entries are contiguous), and a run longer than
// `chunk` entries (chunk >= 64) is cut further into parts of `chunk`.  f(start, end, block) is called
// for every non-empty piece in storage order; returns the number of pieces.  Columns beyond the last
// block (an index out of range) count as the last block.
template <class F>
inline int32_t for_each_piece(const int32_t* rowptr, const uint32_t* idx, int32_t r, int32_t chunk, int32_t block_cols,
                              int32_t max_block, F&& f) {
    const int32_t b = rowptr[r], e = rowptr[r + 1];
    int32_t pieces = 0, k = b;
    while (k < e) {
        int32_t run_end = e, block = 0;
        if (block_cols > 0) {
            block = (int32_t)std::min<uint32_t>((idx[k] & 0x7fffffffu) / (uint32_t)block_cols, (uint32_t)max_block);
            const uint32_t limit = (uint32_t)(block + 1) * (uint32_t)block_cols;       // first column of the next block
            run_end = (int32_t)(std::lower_bound(idx + k, idx + e, limit,
                                                 [](uint32_t v, uint32_t lim) { return (v & 0x7fffffffu) < lim; }) - idx);
            if (run_end <= k) run_end = e;                 // unsorted columns: never stall, keep the rest together
        }
        for (int32_t q = k; q < run_end; q += (chunk > 0 ? chunk : run_end - k)) {
            f(q, chunk > 0 ? std::min(q + chunk, run_end) : run_end, block);
            pieces++;
        }
        k = run_end;
    }
    return pieces;
}

inline int32_t block_columns(int32_t n, int32_t col_blocks) {
    return col_blocks >= 2 ? (int32_t)(((int64_t)n + col_blocks - 1) / col_blocks) : 0;
}

}  // namespace

extern "C" {

void cbm_build_host_timings(double* out4) {
    if (out4) for (int i = 0; i < 4; i++) out4[i] = g_last_timings[i];
}

const char* cbm_host_version(void) { return "cbm4gnn_amd host builder 0.1"; }

void cbm_format_free(cbm_format* f) {
    if (!f) return;
    std::free(f->rowptr); std::free(f->idx); std::free(f->parent); std::free(f->order);
    std::free(f->level_off); std::free(f->mst_row); std::free(f->mst_col);
    std::memset(f, 0, sizeof(*f));
}

int cbm_schedule_rows(const int32_t* rowptr, const int32_t* parent, const float* m, int32_t n,
                      int32_t* sched_out) {
    if (!rowptr || !sched_out) return CBM_ERR_NULL;
    if (n < 0) return CBM_ERR_SHAPE;
    try {
        // counting sort by gather rounds (64 entries each), longest first, stable
        std::vector<int32_t> rounds(n);
        int32_t max_rounds = 0;
        for (int32_t r = 0; r < n; r++) {
            const int32_t len = rowptr[r + 1] - rowptr[r];
            if (len < 0) return CBM_ERR_SHAPE;
            rounds[r] = (len + 63) / 64;
            max_rounds = std::max(max_rounds, rounds[r]);
        }
        std::vector<int64_t> first(max_rounds + 2, 0);
        for (int32_t r = 0; r < n; r++) first[max_rounds - rounds[r] + 1]++;
        for (int32_t b = 0; b <= max_rounds; b++) first[b + 1] += first[b];
        for (int32_t r = 0; r < n; r++) {
            int32_t* o = sched_out + 4 * first[max_rounds - rounds[r]]++;
            const float scale = (m && parent && parent[r] < 0) ? m[r] : 1.0f;
            o[0] = rowptr[r]; o[1] = rowptr[r + 1]; o[2] = r;
            std::memcpy(&o[3], &scale, sizeof(float));
        }
        return CBM_OK;
    } catch (const std::bad_alloc&) {
        return CBM_ERR_ALLOC;
    }
}

int cbm_schedule_rows_batched(const int32_t* rowptr, const int32_t* parent, const float* m, int32_t n,
                              int32_t batch_max_entries, int32_t* sched_out) {
    if (!rowptr || !sched_out) return CBM_ERR_NULL;
    if (n < 0 || batch_max_entries < 0 || batch_max_entries > 64) return CBM_ERR_SHAPE;
    try {
        // sort key, descending, stable: rows above the limit by their 64-entry gather rounds (as
        // cbm_schedule_rows), then the rows of at most `limit` entries by their 8-entry chunks, empty rows last
        const int32_t T = batch_max_entries;
        std::vector<int32_t> key(n);
        int32_t max_key = 0;
        int64_t n_wide = 0;
        for (int32_t r = 0; r < n; r++) {
            const int32_t len = rowptr[r + 1] - rowptr[r];
            if (len < 0) return CBM_ERR_SHAPE;
            if (len > T) { key[r] = 9 + (len + 63) / 64; n_wide++; }
            else key[r] = (len + 7) / 8;                    // 0 .. 8
            max_key = std::max(max_key, key[r]);
        }
        std::vector<int64_t> first(max_key + 2, 0);
        for (int32_t r = 0; r < n; r++) first[max_key - key[r] + 1]++;
        for (int32_t b = 0; b <= max_key; b++) first[b + 1] += first[b];
        for (int32_t r = 0; r < n; r++) {
            int32_t* o = sched_out + 4 * first[max_key - key[r]]++;
            const float scale = (m && parent && parent[r] < 0) ? m[r] : 1.0f;
            o[0] = rowptr[r]; o[1] = rowptr[r + 1]; o[2] = r;
            std::memcpy(&o[3], &scale, sizeof(float));
        }
        int32_t* t = sched_out + 4 * (int64_t)n;            // the trailer
        t[0] = (int32_t)n_wide; t[1] = T; t[2] = CBM_SCHED_BATCH_MAGIC; t[3] = 0;
        return CBM_OK;
    } catch (const std::bad_alloc&) {
        return CBM_ERR_ALLOC;
    }
}

int64_t cbm_schedule_blocks_count(const int32_t* rowptr, const uint32_t* idx, int32_t n, int32_t chunk, int32_t col_blocks,
                                  int32_t* n_long_out) {
    if (!rowptr || n < 0 || (chunk != 0 && chunk < 64) || col_blocks < 0 || (col_blocks >= 2 && !idx && n > 0 && rowptr[n] > 0))
        return -1;
    const int32_t bc = block_columns(n, col_blocks);
    int64_t count = 0;
    int32_t n_long = 0;
    for (int32_t r = 0; r < n; r++) {
        if (rowptr[r + 1] < rowptr[r]) return -1;
        const int32_t pieces = for_each_piece(rowptr, idx, r, chunk, bc, std::max(col_blocks, 1) - 1, [](int32_t, int32_t, int32_t) {});
        if (pieces >= 2) { count += pieces; n_long++; }
        else count++;
    }
    if (n_long_out) *n_long_out = n_long;
    return count;
}

int cbm_schedule_rows_blocks(const int32_t* rowptr, const uint32_t* idx, const int32_t* parent, const float* m, int32_t n,
                             int32_t chunk, int32_t col_blocks, int32_t* sched_out, int32_t* long_rows_out) {
    if (!rowptr || !sched_out) return CBM_ERR_NULL;
    int32_t n_long = 0;
    const int64_t count = cbm_schedule_blocks_count(rowptr, idx, n, chunk, col_blocks, &n_long);
    if (count < 0 || count > INT32_MAX) return CBM_ERR_SHAPE;
    if (n_long > 0 && !long_rows_out) return CBM_ERR_NULL;
    const int32_t bc = block_columns(n, col_blocks);
    try {
        // descriptors of rows and pieces; then a stable counting sort by (column block, descending
        // gather rounds): all wavefronts work on one column block at about the same time, longest first
        struct Item { int32_t start, end, row, block; float scale; };
        std::vector<Item> items;
        items.reserve((size_t)count);
        int32_t slot = 0, at_long = 0;
        std::vector<Item> mine;
        for (int32_t r = 0; r < n; r++) {
            const float scale = (m && parent && parent[r] < 0) ? m[r] : 1.0f;
            mine.clear();
            for_each_piece(rowptr, idx, r, chunk, bc, std::max(col_blocks, 1) - 1,
                           [&](int32_t s, int32_t e, int32_t blk) { mine.push_back({s, e, 0, blk, 1.0f}); });
            if (mine.size() <= 1) {                       // whole row (or an empty one): straight to Z, with its scale
                if (mine.empty()) items.push_back({rowptr[r], rowptr[r + 1], r, 0, scale});
                else items.push_back({mine[0].start, mine[0].end, r, mine[0].block, scale});
                continue;
            }
            int32_t* lr = long_rows_out + 4 * (size_t)at_long++;
            lr[0] = r; lr[1] = slot; lr[2] = (int32_t)mine.size();
            std::memcpy(&lr[3], &scale, sizeof(float));
            for (Item& it : mine) { it.row = (slot++) | CBM_SCHED_PIECE; items.push_back(it); }
        }
        int32_t max_rounds = 0;
        for (const Item& it : items) max_rounds = std::max(max_rounds, (it.end - it.start + 63) / 64);
        const int64_t n_blocks = std::max(col_blocks, 1), buckets = n_blocks * (max_rounds + 1);
        std::vector<int64_t> first((size_t)buckets + 1, 0);
        auto bucket = [&](const Item& it) {
            return (int64_t)it.block * (max_rounds + 1) + (max_rounds - (it.end - it.start + 63) / 64);
        };
        for (const Item& it : items) first[bucket(it) + 1]++;
        for (int64_t b = 0; b < buckets; b++) first[b + 1] += first[b];
        for (const Item& it : items) {
            int32_t* o = sched_out + 4 * first[bucket(it)]++;
            o[0] = it.start; o[1] = it.end; o[2] = it.row;
            std::memcpy(&o[3], &it.scale, sizeof(float));
        }
        return CBM_OK;
    } catch (const std::bad_alloc&) {
        return CBM_ERR_ALLOC;
    }
}

int64_t cbm_schedule_split_count(const int32_t* rowptr, int32_t n, int32_t chunk, int32_t* n_long_out) {
    if (chunk < 64) return -1;
    return cbm_schedule_blocks_count(rowptr, nullptr, n, chunk, 1, n_long_out);
}

int cbm_schedule_rows_split(const int32_t* rowptr, const int32_t* parent, const float* m, int32_t n, int32_t chunk,
                            int32_t* sched_out, int32_t* long_rows_out) {
    if (chunk < 64) return CBM_ERR_SHAPE;
    return cbm_schedule_rows_blocks(rowptr, nullptr, parent, m, n, chunk, 1, sched_out, long_rows_out);
}

void cbm_walk_plan_free(cbm_walk_plan* p) {
    if (!p) return;
    free(p->entries); free(p->bin_off);
    std::memset(p, 0, sizeof(*p));
}

}  // extern "C"

namespace {

// The arborescence as child lists, for the plans that walk it depth-first.
struct WalkTree {
    std::vector<int32_t> level, child_ptr, child, size;

    // Validates parent / order / level_off against each other and builds the child lists, lightest subtree
    // first (ties by id): the value of a row then has to be kept only while the walk is inside one of its
    // lighter children, which bounds the kept values by log2(subtree size).
    int build(const int32_t* parent, const int32_t* order, const int32_t* level_off, int32_t n, int32_t n_levels) {
        if (level_off[0] != 0 || level_off[n_levels] != n) return CBM_ERR_SHAPE;
        for (int32_t l = 0; l < n_levels; l++)
            if (level_off[l + 1] < level_off[l]) return CBM_ERR_SHAPE;
        // level of every row; order must be a permutation whose rows sit one level below their parents
        level.assign(n, -1);
        for (int32_t l = 0; l < n_levels; l++)
            for (int32_t i = level_off[l]; i < level_off[l + 1]; i++) {
                const int32_t v = order[i];
                if (v < 0 || v >= n || level[v] >= 0) return CBM_ERR_SHAPE;
                level[v] = l;
            }
        for (int32_t v = 0; v < n; v++) {
            const int32_t u = parent[v];
            if (u >= n || u == v) return CBM_ERR_SHAPE;
            if (u < 0 ? level[v] != 0 : level[u] + 1 != level[v]) return CBM_ERR_SHAPE;
        }
        // children lists (CSR by parent) and subtree sizes (leaves first: order[] backwards)
        child_ptr.assign(n + 1, 0);
        child.assign(n > 0 ? n : 1, 0);
        size.assign(n, 1);
        for (int32_t v = 0; v < n; v++)
            if (parent[v] >= 0) child_ptr[parent[v] + 1]++;
        for (int32_t v = 0; v < n; v++) child_ptr[v + 1] += child_ptr[v];
        {
            std::vector<int32_t> at(child_ptr.begin(), child_ptr.end() - 1);
            for (int32_t v = 0; v < n; v++)
                if (parent[v] >= 0) child[at[parent[v]]++] = v;
        }
        for (int32_t i = n - 1; i >= 0; i--) {
            const int32_t v = order[i];
            if (parent[v] >= 0) size[parent[v]] += size[v];
        }
        for (int32_t v = 0; v < n; v++)
            std::sort(child.begin() + child_ptr[v], child.begin() + child_ptr[v + 1],
                      [&](int32_t a, int32_t b) { return size[a] != size[b] ? size[a] < size[b] : a < b; });
        return CBM_OK;
    }

    // The subtree of r in depth-first pre-order as { row, ctl } pairs (ctl as in struct cbm_walk_plan), handed
    // to put(row, ctl) one by one.  False if a row would need more than CBM_WALK_MAX_SLOTS kept values.
    template <class Put>
    bool emit(int32_t r, int32_t& max_slots, Put put) {
        int32_t kept = 0;                                  // rows on the current path whose value sits in a slot
        {
            int32_t ctl = CBM_WALK_LOAD_ONLY;
            if (child_ptr[r + 1] - child_ptr[r] >= 2) { kept++; ctl |= kept << 8; }
            put(r, ctl);
        }
        stack.clear();
        slot_of_depth.clear();
        stack.emplace_back(r, 0);
        slot_of_depth.push_back(kept);                     // slot of the stack's rows (0 = none)
        max_slots = std::max(max_slots, kept);
        while (!stack.empty()) {
            const int32_t u = stack.back().first;
            const int32_t i = stack.back().second;
            const int32_t k = child_ptr[u + 1] - child_ptr[u];
            if (i == k) { stack.pop_back(); slot_of_depth.pop_back(); continue; }
            stack.back().second = i + 1;
            const int32_t v = child[child_ptr[u] + i];
            // source of the parent's value: the row visited just before (first child), else the parent's slot;
            // the last child frees that slot before taking one of its own
            int32_t ctl = (i == 0) ? 0 : slot_of_depth.back();
            if (i == k - 1 && k >= 2) kept--;
            const int32_t kv = child_ptr[v + 1] - child_ptr[v];
            int32_t mine = 0;
            if (kv >= 2) {
                mine = ++kept;
                if (mine > CBM_WALK_MAX_SLOTS) return false;
                max_slots = std::max(max_slots, mine);
                ctl |= mine << 8;
            }
            put(v, ctl);
            if (kv > 0) { stack.emplace_back(v, 0); slot_of_depth.push_back(mine); }
        }
        return true;
    }

private:
    std::vector<std::pair<int32_t, int32_t>> stack;        // (row, next child to visit)
    std::vector<int32_t> slot_of_depth;
};

}  // namespace

extern "C" {

int cbm_walk_plan_build(const int32_t* parent, const int32_t* order, const int32_t* level_off, int32_t n,
                        int32_t n_levels, int32_t cut, int32_t target_bins, cbm_walk_plan* out) {
    if (!out) return CBM_ERR_NULL;
    std::memset(out, 0, sizeof(*out));
    if (!parent || !order || !level_off) return CBM_ERR_NULL;
    if (n <= 0 || n_levels < 1 || cut < 0 || cut >= n_levels || target_bins < 1) return CBM_ERR_SHAPE;
    try {
        WalkTree tree;
        if (int rc = tree.build(parent, order, level_off, n, n_levels)) return rc;
        const std::vector<int32_t>& size = tree.size;
        // tasks: the rows of level `cut` that have children, longest subtree first (ties by id)
        std::vector<int32_t> roots;
        for (int32_t i = level_off[cut]; i < level_off[cut + 1]; i++)
            if (size[order[i]] > 1) roots.push_back(order[i]);
        std::sort(roots.begin(), roots.end(),
                  [&](int32_t a, int32_t b) { return size[a] != size[b] ? size[a] > size[b] : a < b; });
        int64_t total = 0;
        for (int32_t r : roots) total += size[r];
        if (total > INT32_MAX) return CBM_ERR_SHAPE;
        out->n = n; out->cut = cut; out->n_entries = (int32_t)total;
        out->entries = (int32_t*)malloc(sizeof(int32_t) * 2 * std::max<size_t>((size_t)total, 1));
        if (!out->entries) throw std::bad_alloc();
        // bins: consecutive tasks of the sorted list until a bin holds `target` entries
        const int64_t target = std::max<int64_t>((total + target_bins - 1) / target_bins, CBM_WALK_MIN_BIN);
        std::vector<int32_t> bin_off(1, 0);
        int64_t at = 0, in_bin = 0, longest = 0;
        int32_t max_slots = 0;
        for (int32_t r : roots) {
            if (in_bin >= target) { bin_off.push_back((int32_t)at); longest = std::max(longest, in_bin); in_bin = 0; }
            in_bin += size[r];
            const bool fits = tree.emit(r, max_slots, [&](int32_t row, int32_t ctl) {
                out->entries[2 * at] = row; out->entries[2 * at + 1] = ctl;
                at++;
            });
            if (!fits) return (cbm_walk_plan_free(out), CBM_ERR_UNSUPPORTED);
        }
        if (at != total) return (cbm_walk_plan_free(out), CBM_ERR_INTERNAL);
        if (total > 0) { bin_off.push_back((int32_t)at); longest = std::max(longest, in_bin); }
        out->n_bins = (int32_t)bin_off.size() - 1;
        out->n_slots = max_slots;
        out->longest_bin = longest;
        out->bin_off = (int32_t*)malloc(sizeof(int32_t) * bin_off.size());
        if (!out->bin_off) throw std::bad_alloc();
        std::copy(bin_off.begin(), bin_off.end(), out->bin_off);
        return CBM_OK;
    } catch (const std::bad_alloc&) {
        cbm_walk_plan_free(out);
        return CBM_ERR_ALLOC;
    }
}

void cbm_walk_stream_free(cbm_walk_stream* p) {
    if (!p) return;
    free(p->gidx); free(p->ginfo); free(p->bin_goff);
    std::memset(p, 0, sizeof(*p));
}

int cbm_walk_stream_build(const int32_t* rowptr, const uint32_t* idx, const int32_t* parent, const int32_t* order,
                          const int32_t* level_off, int32_t n, int32_t n_levels, int32_t target_bins,
                          cbm_walk_stream* out) {
    if (!out) return CBM_ERR_NULL;
    std::memset(out, 0, sizeof(*out));
    if (!rowptr || !parent || !order || !level_off) return CBM_ERR_NULL;
    if (n <= 0 || n_levels < 1 || target_bins < 1 || (uint32_t)n > CBM_STREAM_COL_MASK) return CBM_ERR_SHAPE;
    if (rowptr[0] != 0) return CBM_ERR_SHAPE;
    for (int32_t r = 0; r < n; r++)
        if (rowptr[r + 1] < rowptr[r]) return CBM_ERR_SHAPE;
    if (rowptr[n] > 0 && !idx) return CBM_ERR_NULL;
    for (int64_t k = 0; k < rowptr[n]; k++)
        if ((idx[k] & 0x7fffffffu) >= (uint32_t)n) return CBM_ERR_SHAPE;
    try {
        WalkTree tree;
        if (int rc = tree.build(parent, order, level_off, n, n_levels)) return rc;
        // a row costs its delta entries (an empty row one stand-in entry) + CBM_STREAM_ROW_COST for its walk
        // step and store; a subtree the sum over its rows
        std::vector<int64_t> weight(n);
        int64_t total = 0;
        for (int32_t v = 0; v < n; v++) total += weight[v] = std::max(rowptr[v + 1] - rowptr[v], 1) + CBM_STREAM_ROW_COST;
        if (total > INT32_MAX) return CBM_ERR_SHAPE;
        for (int32_t i = n - 1; i >= 0; i--) {
            const int32_t v = order[i];
            if (parent[v] >= 0) weight[parent[v]] += weight[v];
        }
        // tasks: every child of the root, heaviest subtree first (ties by id)
        std::vector<int32_t> roots(order, order + level_off[1]);
        std::sort(roots.begin(), roots.end(),
                  [&](int32_t a, int32_t b) { return weight[a] != weight[b] ? weight[a] > weight[b] : a < b; });
        // bins: consecutive tasks of the sorted list until a bin weighs `target`
        const int64_t target = std::max<int64_t>((total + target_bins - 1) / target_bins, CBM_STREAM_MIN_BIN);
        std::vector<int32_t> entries;                      // { row, ctl } in walk order
        entries.reserve(2 * (size_t)n);
        std::vector<int32_t> bin_first(1, 0);              // first row (position in entries) of every bin
        int64_t in_bin = 0, heaviest = 0;
        int32_t max_slots = 0;
        for (int32_t r : roots) {
            if (in_bin >= target) { bin_first.push_back((int32_t)(entries.size() / 2)); in_bin = 0; }
            in_bin += weight[r];
            heaviest = std::max(heaviest, in_bin);
            if (!tree.emit(r, max_slots, [&](int32_t row, int32_t ctl) { entries.push_back(row); entries.push_back(ctl); }))
                return CBM_ERR_UNSUPPORTED;
        }
        if (entries.size() != 2 * (size_t)n) return CBM_ERR_INTERNAL;
        bin_first.push_back(n);
        const int32_t n_bins = (int32_t)bin_first.size() - 1;
        // every bin is padded to whole stretches of 64 entries (the kernel never tests for the end of a bin
        // inside a stretch): copies of its last entry without marks, whose sum goes nowhere
        std::vector<int64_t> goff(n_bins + 1, 0);
        for (int32_t b = 0; b < n_bins; b++) {
            int64_t elems = 0;
            for (int32_t k = bin_first[b]; k < bin_first[b + 1]; k++) {
                const int32_t row = entries[2 * (size_t)k];
                elems += std::max(rowptr[row + 1] - rowptr[row], 1);
            }
            goff[b + 1] = goff[b] + (elems + 63) / 64 * 64;
        }
        const int64_t padded = goff[n_bins];
        if (padded > INT32_MAX) return CBM_ERR_SHAPE;
        out->n = n; out->n_bins = n_bins; out->n_slots = max_slots; out->n_elems = (int32_t)padded;
        out->gidx = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)padded);
        out->ginfo = (int32_t*)calloc(2 * (size_t)padded, sizeof(int32_t));   // zeroed: "no row landed here"
        out->bin_goff = (int32_t*)malloc(sizeof(int32_t) * ((size_t)n_bins + 1));
        if (!out->gidx || !out->ginfo || !out->bin_goff) throw std::bad_alloc();
        for (int32_t b = 0; b < n_bins; b++) {
            const int64_t g0 = goff[b];
            int64_t g = g0;
            out->bin_goff[b] = (int32_t)g0;
            int64_t stretch = -1;
            int32_t in_stretch = 0;
            for (int32_t k = bin_first[b]; k < bin_first[b + 1]; k++) {
                const int32_t row = entries[2 * (size_t)k], ctl = entries[2 * (size_t)k + 1];
                const int32_t len = rowptr[row + 1] - rowptr[row];
                if (len == 0) {
                    out->gidx[g++] = (uint32_t)row | CBM_STREAM_DUMMY | CBM_STREAM_LAST;
                } else {
                    for (int32_t e = 0; e < len; e++) out->gidx[g++] = idx[rowptr[row] + e];
                    out->gidx[g - 1] |= CBM_STREAM_LAST;
                }
                // the rows that end inside a stretch of 64 entries, in order, sit at the head of that stretch
                const int64_t s = (g - 1 - g0) / 64;
                if (s != stretch) { stretch = s; in_stretch = 0; }
                int32_t* info = out->ginfo + 2 * (g0 + s * 64 + in_stretch++);
                info[0] = row; info[1] = ctl | INT32_MIN;  // marked: a slot that is in use
            }
            const uint32_t pad = out->gidx[g - 1] & CBM_STREAM_COL_MASK;
            while (g < goff[b + 1]) out->gidx[g++] = pad;
            // slots no row landed in: a valid row (the kernel loads them, and m of their row, without using them)
            const int32_t filler = entries[2 * (size_t)bin_first[b]];
            for (int64_t q = g0; q < g; q++) {
                int32_t* info = out->ginfo + 2 * q;
                if (info[1] < 0) info[1] &= INT32_MAX;
                else { info[0] = filler; info[1] = 0; }
            }
        }
        out->bin_goff[n_bins] = (int32_t)padded;
        out->heaviest_bin = heaviest;
        return CBM_OK;
    } catch (const std::bad_alloc&) {
        cbm_walk_stream_free(out);
        return CBM_ERR_ALLOC;
    }
}

void cbm_tiling_free(cbm_tiling* t) {
    if (!t) return;
    free(t->panel_ptr); free(t->blk_tile); free(t->seg); free(t->lidx); free(t->rowptr_r); free(t->idx_r);
    std::memset(t, 0, sizeof(*t));
}

int cbm_tile_rows(const int32_t* rowptr, const uint32_t* idx, int32_t n, int32_t tile_rows, int64_t min_block_entries,
                  int32_t threads, cbm_tiling* out) {
    if (!out) return CBM_ERR_NULL;
    std::memset(out, 0, sizeof(*out));
    if (n < 0 || (tile_rows != 1024 && tile_rows != 512) || min_block_entries < 1) return CBM_ERR_SHAPE;
    if (!rowptr || (n > 0 && rowptr[n] > 0 && !idx)) return CBM_ERR_NULL;
    if (threads <= 0) threads = omp_get_max_threads();
    constexpr int P = CBM_TILING_PANEL_ROWS;
    const int T = tile_rows;
    const int32_t n_panels = (n + P - 1) / P, n_tiles = (n + T - 1) / T;
    for (int32_t r = 0; r < n; r++)
        if (rowptr[r + 1] < rowptr[r]) return CBM_ERR_SHAPE;
    try {
        // pass 1: per panel, the tiles that hold at least min_block_entries of its entries
        std::vector<std::vector<int32_t>> tiles_of(n_panels);
        // (a std::bad_alloc must not leave a parallel region: caught inside, flagged, rethrown after it)
        int bad = 0, no_memory = 0;
#pragma omp parallel num_threads(threads)
        {
            try {
                std::vector<int64_t> cnt(n_tiles, 0);
                std::vector<int32_t> touched;
#pragma omp for schedule(dynamic, 4)
                for (int32_t p = 0; p < n_panels; p++) {
                    touched.clear();
                    const int32_t r_end = std::min<int64_t>((int64_t)(p + 1) * P, n);
                    int wrong = 0;
                    for (int32_t r = p * P; r < r_end; r++) {
                        int64_t before = -1;                // columns must ascend inside a row: the fill below
                        for (int64_t k = rowptr[r]; k < rowptr[r + 1]; k++) {   // takes a block's entries as one run
                            const uint32_t c = idx[k] & 0x7fffffffu;
                            if (c >= (uint32_t)n || (int64_t)c <= before) { wrong = 1; continue; }
                            before = c;
                            const int32_t t = (int32_t)(c / (uint32_t)T);
                            if (cnt[t]++ == 0) touched.push_back(t);
                        }
                    }
                    if (wrong) {
#pragma omp atomic write
                        bad = 1;
                    }
                    std::sort(touched.begin(), touched.end());
                    for (int32_t t : touched) {
                        if (cnt[t] >= min_block_entries) tiles_of[p].push_back(t);
                        cnt[t] = 0;
                    }
                }
            } catch (const std::bad_alloc&) {
#pragma omp atomic write
                no_memory = 1;
            }
        }
        if (no_memory) throw std::bad_alloc();
        if (bad) return CBM_ERR_SHAPE;
        out->n = n; out->tile_rows = T; out->panel_rows = P; out->n_panels = n_panels;
        out->panel_ptr = (int32_t*)malloc(sizeof(int32_t) * ((size_t)n_panels + 1));
        if (!out->panel_ptr) throw std::bad_alloc();
        out->panel_ptr[0] = 0;
        for (int32_t p = 0; p < n_panels; p++) out->panel_ptr[p + 1] = out->panel_ptr[p] + (int32_t)tiles_of[p].size();
        const int32_t B = out->panel_ptr[n_panels];
        out->n_blocks = B;
        out->blk_tile = (int32_t*)malloc(sizeof(int32_t) * std::max<size_t>(B, 1));
        out->seg = (int32_t*)malloc(sizeof(int32_t) * std::max<size_t>((size_t)B * (P + 1), 1));
        out->rowptr_r = (int32_t*)malloc(sizeof(int32_t) * ((size_t)n + 1));
        if (!out->blk_tile || !out->seg || !out->rowptr_r) throw std::bad_alloc();
        for (int32_t p = 0; p < n_panels; p++)
            std::copy(tiles_of[p].begin(), tiles_of[p].end(), out->blk_tile + out->panel_ptr[p]);
        // pass 2: entries per (block, panel row) -> seg (as counts first), remote entries per row
        std::fill(out->seg, out->seg + (size_t)B * (P + 1), 0);
        int any_negative = 0;
#pragma omp parallel num_threads(threads)
        {
            std::vector<int32_t> block_of;
            try { block_of.assign(n_tiles, -1); } catch (const std::bad_alloc&) {
#pragma omp atomic write
                no_memory = 1;
            }
            int neg = 0;
            const bool usable = (int32_t)block_of.size() == n_tiles;
#pragma omp for schedule(dynamic, 4)
            for (int32_t p = 0; p < n_panels; p++) {
                if (!usable) continue;
                const int32_t b0 = out->panel_ptr[p];
                for (size_t i = 0; i < tiles_of[p].size(); i++) block_of[tiles_of[p][i]] = b0 + (int32_t)i;
                const int32_t r_end = std::min<int64_t>((int64_t)(p + 1) * P, n);
                for (int32_t r = p * P; r < r_end; r++) {
                    int32_t remote = 0;
                    for (int64_t k = rowptr[r]; k < rowptr[r + 1]; k++) {
                        const int32_t b = block_of[(idx[k] & 0x7fffffffu) / (uint32_t)T];
                        if (b >= 0) { out->seg[(size_t)b * (P + 1) + (r - p * P)]++; neg |= (int)(idx[k] >> 31); }
                        else remote++;
                    }
                    out->rowptr_r[r + 1] = remote;
                }
                for (int32_t t : tiles_of[p]) block_of[t] = -1;
            }
            if (neg) {
#pragma omp atomic write
                any_negative = 1;
            }
        }
        if (no_memory) throw std::bad_alloc();
        // counts -> offsets: segments padded to multiples of 8 entries, seg[] in units of 8 entries
        int64_t at8 = 0, real = 0;
        for (int32_t b = 0; b < B; b++) {
            int32_t* sg = out->seg + (size_t)b * (P + 1);
            for (int pr = 0; pr < P; pr++) {
                const int32_t c = sg[pr];
                real += c;
                sg[pr] = (int32_t)at8;
                at8 += (c + 7) / 8;
                if (at8 > INT32_MAX) return (cbm_tiling_free(out), CBM_ERR_SHAPE);
            }
            sg[P] = (int32_t)at8;
        }
        out->rowptr_r[0] = 0;
        for (int32_t r = 0; r < n; r++) out->rowptr_r[r + 1] += out->rowptr_r[r];
        out->nnz_local = real;
        out->nnz_local_padded = at8 * 8;
        out->nnz_remote = n > 0 ? out->rowptr_r[n] : 0;
        out->has_negative = any_negative;
        out->lidx = (uint16_t*)malloc(sizeof(uint16_t) * std::max<size_t>((size_t)at8 * 8, 8));
        out->idx_r = (uint32_t*)malloc(sizeof(uint32_t) * std::max<size_t>((size_t)out->nnz_remote, 1));
        if (!out->lidx || !out->idx_r) throw std::bad_alloc();
        // pass 3: fill.  A local entry is (row of X - first row of its tile) * 8 | sign << 15; the padding
        // of a segment names row T, the all-zero row the kernel keeps behind the tile.
        const uint16_t pad = (uint16_t)(T * 8);
#pragma omp parallel num_threads(threads)
        {
            std::vector<int32_t> block_of;
            try { block_of.assign(n_tiles, -1); } catch (const std::bad_alloc&) {
#pragma omp atomic write
                no_memory = 1;
            }
            const bool usable = (int32_t)block_of.size() == n_tiles;
#pragma omp for schedule(dynamic, 4)
            for (int32_t p = 0; p < n_panels; p++) {
                if (!usable) continue;
                const int32_t b0 = out->panel_ptr[p];
                for (size_t i = 0; i < tiles_of[p].size(); i++) block_of[tiles_of[p][i]] = b0 + (int32_t)i;
                const int32_t r_end = std::min<int64_t>((int64_t)(p + 1) * P, n);
                for (size_t i = 0; i < tiles_of[p].size(); i++) {       // padding first, entries overwrite it
                    const int32_t* sg = out->seg + (size_t)(b0 + i) * (P + 1);
                    std::fill(out->lidx + (size_t)sg[0] * 8, out->lidx + (size_t)sg[P] * 8, pad);
                }
                for (int32_t r = p * P; r < r_end; r++) {
                    int64_t at_r = out->rowptr_r[r];
                    // Columns ascend within a row, so the entries of one block form one run.  Inside a
                    // segment the entries are stored by the class q = (column - row) mod 4, in the order
                    // q = 0, 2, 1, 3, ascending inside a class.  A 128-byte row of the tile covers half of
                    // the LDS banks, chosen by the parity of its index, and the kernel serves two
                    // neighbouring matrix rows per cycle: with q = 0, 2 first a row of even index reads even
                    // columns first and its odd neighbour odd ones -- opposite halves nearly always.  A
                    // 64-byte row (the half slab) covers a quarter of the banks, chosen by its index mod 4,
                    // and four neighbouring matrix rows are served per cycle: in step they read the four
                    // different classes.
                    int64_t k = rowptr[r];
                    const int64_t k_end = rowptr[r + 1];
                    while (k < k_end) {
                        const uint32_t c0 = idx[k] & 0x7fffffffu;
                        const int32_t t = (int32_t)(c0 / (uint32_t)T);
                        const int32_t b = block_of[t];
                        if (b < 0) { out->idx_r[at_r++] = idx[k++]; continue; }
                        int64_t k1 = k;
                        while (k1 < k_end && (int32_t)((idx[k1] & 0x7fffffffu) / (uint32_t)T) == t) k1++;
                        int64_t at = (int64_t)out->seg[(size_t)b * (P + 1) + (r - p * P)] * 8;
                        static const uint32_t kClassOrder[4] = {0u, 2u, 1u, 3u};
                        for (int pass = 0; pass < 4; pass++)
                            for (int64_t q = k; q < k1; q++) {
                                const uint32_t c = idx[q] & 0x7fffffffu;
                                if (((c - (uint32_t)r) & 3u) != kClassOrder[pass]) continue;
                                out->lidx[at++] = (uint16_t)(((c - (uint32_t)t * (uint32_t)T) * 8u) | ((idx[q] >> 31) << 15));
                            }
                        k = k1;
                    }
                }
                for (int32_t t : tiles_of[p]) block_of[t] = -1;
            }
        }
        if (no_memory) throw std::bad_alloc();
        return CBM_OK;
    } catch (const std::bad_alloc&) {
        cbm_tiling_free(out);
        return CBM_ERR_ALLOC;
    }
}

int cbm_builder_create(const int32_t* row, const int32_t* col, int64_t E, int32_t N, int32_t threads,
                       cbm_builder** out) {
    if (!out) return CBM_ERR_NULL;
    *out = nullptr;
    if ((!row || !col) && E > 0) return CBM_ERR_NULL;
    if (N <= 0 || E < 0 || N >= (1 << 30)) return CBM_ERR_SHAPE;
    if (threads <= 0) threads = omp_get_max_threads();
    const double t0 = omp_get_wtime();
    cbm_builder* b = nullptr;
    try {
        b = new cbm_builder();
        b->threads = threads;
        if (int rc = build_graph(row, col, E, N, threads, b->g)) { delete b; return rc; }
    } catch (const std::bad_alloc&) {
        delete b;
        return CBM_ERR_ALLOC;
    }
    g_last_timings[0] = omp_get_wtime() - t0;
    g_last_timings[1] = g_last_timings[2] = g_last_timings[3] = 0;
    *out = b;
    return CBM_OK;
}

int cbm_builder_arrays(const cbm_builder* b, const int64_t** rowptr, const int32_t** col, const int64_t** colptr_t,
                       const int32_t** row_t, const int64_t** after, const int32_t** row_nnz, int64_t* nnz) {
    if (!b) return CBM_ERR_NULL;
    if (rowptr) *rowptr = b->g.rp.data();
    if (col) *col = b->g.ci.data();
    if (colptr_t) *colptr_t = b->g.tp.data();
    if (row_t) *row_t = b->g.tr.data();
    if (after) *after = b->g.after.data();
    if (row_nnz) *row_nnz = b->g.nnz.data();
    if (nnz) *nnz = b->g.nnzA;
    return CBM_OK;
}

int cbm_builder_finish(cbm_builder* b, int32_t alpha, const cbm_pair* pairs, int64_t n_pairs, cbm_format* out) {
    if (!out) return CBM_ERR_NULL;
    std::memset(out, 0, sizeof(*out));
    if (!b || (n_pairs > 0 && !pairs)) return CBM_ERR_NULL;
    const double t0 = omp_get_wtime();
    try {
        std::vector<CandEdge> cand;
        const int rc = n_pairs < 0 ? candidates_host(b->g, alpha, b->threads, cand)
                                   : candidates_from_pairs(b->g, alpha, pairs, n_pairs, b->threads, cand);
        if (rc) return rc;
        const double t1 = omp_get_wtime();
        g_last_timings[1] = t1 - t0;
        return finish_format(b->g, cand, b->threads, b->max_levels, out, t1);
    } catch (const std::bad_alloc&) {
        cbm_format_free(out);
        return CBM_ERR_ALLOC;
    }
}

int cbm_builder_set_max_levels(cbm_builder* b, int32_t max_levels) {
    if (!b) return CBM_ERR_NULL;
    if (max_levels < 0) return CBM_ERR_SHAPE;
    b->max_levels = max_levels;
    return CBM_OK;
}

void cbm_builder_free(cbm_builder* b) { delete b; }

int cbm_build_host(const int32_t* row, const int32_t* col, int64_t E, int32_t N, int32_t alpha,
                   int32_t threads, cbm_format* out) {
    if (!out) return CBM_ERR_NULL;
    std::memset(out, 0, sizeof(*out));
    cbm_builder* b = nullptr;
    if (int rc = cbm_builder_create(row, col, E, N, threads, &b)) return rc;
    const int rc = cbm_builder_finish(b, alpha, nullptr, -1, out);
    cbm_builder_free(b);
    return rc;
}

}  // extern "C"
