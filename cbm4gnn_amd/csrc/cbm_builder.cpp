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
//     (meldable leftist heaps with lazy keys, union-find with rollback for the expansion).
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

// ---------------------------------------------------------------------------------------------
// Minimum spanning arborescence (Tarjan 1977 / Camerini-Fratta-Maffioli 1979 expansion).
// ---------------------------------------------------------------------------------------------
class Arborescence {
public:
    Arborescence(int32_t n, const std::vector<CandEdge>& edges, int threads)
        : n_(n), threads_(threads), edges_(edges), node_(edges.size()), heap_(n, -1), uf_(n, -1) {}

    // Returns total weight; par[v] = tail of the edge entering v (par[root] = -1).
    int64_t run(int32_t root, std::vector<int32_t>& par) {
        const int64_t m = (int64_t)edges_.size();
        // One heap per head node, built without a single meld: the node's incoming edges sorted
        // by (weight, id) and chained through the LEFT child is a valid leftist heap (every right
        // child is empty), and the sorts run in parallel.
        {
            std::vector<int64_t> cnt(n_ + 1, 0);
            for (int64_t e = 0; e < m; e++) cnt[edges_[e].v + 1]++;
            for (int32_t v = 0; v < n_; v++) cnt[v + 1] += cnt[v];
            std::vector<int32_t> ids(m);
            {
                std::vector<int64_t> fill(cnt.begin(), cnt.end() - 1);
                for (int64_t e = 0; e < m; e++) ids[fill[edges_[e].v]++] = (int32_t)e;
            }
#pragma omp parallel for schedule(dynamic, 64) num_threads(threads_)
            for (int32_t v = 0; v < n_; v++) {
                const int64_t b = cnt[v], e = cnt[v + 1];
                if (b == e) continue;
                std::sort(ids.begin() + b, ids.begin() + e, [&](int32_t x, int32_t y) {
                    return edges_[x].w != edges_[y].w ? edges_[x].w < edges_[y].w : x < y;
                });
                for (int64_t k = b; k < e; k++) {
                    Node& nd = node_[ids[k]];
                    nd.key = edges_[ids[k]].w; nd.lazy = 0;
                    nd.lc = k + 1 < e ? ids[k + 1] : -1; nd.rc = -1; nd.rank = 1;
                }
                heap_[v] = ids[b];
            }
        }
        std::vector<int32_t> seen(n_, -1), path(n_), Q(n_), in(n_, -1);
        seen[root] = root;
        int64_t res = 0;
        struct Cycle { int32_t node; int32_t time; int32_t eb, ee; };
        std::vector<Cycle> cycles;
        std::vector<int32_t> cyc_edges;
        for (int32_t s = 0; s < n_; s++) {
            int32_t u = s, qi = 0;
            while (seen[u] < 0) {
                int32_t h = heap_[u];
                if (h < 0) return -1;                   // node not reachable from the root
                push_down(h);
                const int32_t e = h;
                const int32_t w = node_[e].key;
                heap_[u] = meld(node_[e].lc, node_[e].rc);            // pop
                // An edge inside the (contracted) component is dropped outright.  Charging its
                // reduced weight and discounting the rest of the heap by it, as for any other
                // popped edge, would cancel out with the next pop of this heap, and the one-edge
                // "cycle" it would record expands to nothing.
                if (find(edges_[e].u) == u) continue;
                if (heap_[u] >= 0) node_[heap_[u]].lazy -= w;        // remaining keys become reduced costs
                Q[qi] = e; path[qi++] = u; seen[u] = s;
                res += w;
                u = find(edges_[e].u);
                if (seen[u] == s) {                      // closed a cycle: contract it into u
                    int32_t cyc = -1;
                    const int32_t end = qi, time = (int32_t)hist_.size();
                    int32_t x;
                    do { x = path[--qi]; cyc = meld(cyc, heap_[x]); } while (join(u, x));
                    u = find(u);
                    heap_[u] = cyc; seen[u] = -1;
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
    struct Node { int32_t key, lazy, lc, rc; int32_t rank; };   // one cache line holds three
    int32_t n_;
    int threads_;
    const std::vector<CandEdge>& edges_;
    std::vector<Node> node_;                                   // index = edge id
    std::vector<int32_t> heap_;
    std::vector<int32_t> uf_;                                  // <0: -size, else parent
    std::vector<std::pair<int32_t, int32_t>> hist_;

    void push_down(int32_t a) {
        Node& nd = node_[a];
        const int32_t z = nd.lazy;
        if (z) {
            nd.key += z;
            if (nd.lc >= 0) node_[nd.lc].lazy += z;
            if (nd.rc >= 0) node_[nd.rc].lazy += z;
            nd.lazy = 0;
        }
    }
    // Leftist heap meld; the right spine is O(log size) so the recursion is shallow.  Ties are
    // broken towards the smaller edge id, which makes the result independent of meld order.
    int32_t meld(int32_t a, int32_t b) {
        if (a < 0) return b;
        if (b < 0) return a;
        push_down(a); push_down(b);
        if (node_[a].key > node_[b].key || (node_[a].key == node_[b].key && a > b)) std::swap(a, b);
        Node& na = node_[a];
        na.rc = meld(na.rc, b);
        const int32_t rl = na.lc >= 0 ? node_[na.lc].rank : 0, rr = node_[na.rc].rank;
        if (rl < rr) std::swap(na.lc, na.rc);
        na.rank = (na.rc >= 0 ? node_[na.rc].rank : 0) + 1;
        return a;
    }
    int32_t find(int32_t x) const { while (uf_[x] >= 0) x = uf_[x]; return x; }
    bool join(int32_t a, int32_t b) {
        a = find(a); b = find(b);
        if (a == b) return false;
        if (uf_[a] > uf_[b]) std::swap(a, b);
        hist_.push_back({a, uf_[a]}); hist_.push_back({b, uf_[b]});
        uf_[a] += uf_[b]; uf_[b] = a;
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

}  // namespace

// seconds spent by the last cbm_build_host call of this thread in: CSR + transpose, candidate
// edges, arborescence, tree arrays + deltas
thread_local double g_last_timings[4] = {0, 0, 0, 0};

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

int cbm_build_host(const int32_t* row, const int32_t* col, int64_t E, int32_t N, int32_t alpha,
                   int32_t threads, cbm_format* out) {
    if (!out) return CBM_ERR_NULL;
    std::memset(out, 0, sizeof(*out));
    if ((!row || !col) && E > 0) return CBM_ERR_NULL;
    if (N <= 0 || E < 0 || N >= (1 << 30)) return CBM_ERR_SHAPE;
    if (threads <= 0) threads = omp_get_max_threads();
    double t_mark = omp_get_wtime();
    auto lap = [&](int slot) { const double t = omp_get_wtime(); g_last_timings[slot] = t - t_mark; t_mark = t; };
    try {
        // ---- COO -> CSR(A) with sorted unique columns, and its transpose -----------------------
        std::vector<int64_t> rp(N + 1, 0);
        for (int64_t k = 0; k < E; k++) {
            if (row[k] < 0 || row[k] >= N || col[k] < 0 || col[k] >= N) return CBM_ERR_SHAPE;
            rp[row[k] + 1]++;
        }
        for (int32_t r = 0; r < N; r++) rp[r + 1] += rp[r];
        std::vector<int32_t> ci(E);
        {
            std::vector<int64_t> fill(rp.begin(), rp.end() - 1);
            for (int64_t k = 0; k < E; k++) ci[fill[row[k]]++] = col[k];
        }
        std::vector<int32_t> nnz(N);
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
        const int64_t nnzA = rp[N];
        std::vector<int64_t> tp(N + 1, 0);
        for (int64_t k = 0; k < nnzA; k++) tp[ci[k] + 1]++;
        for (int32_t c = 0; c < N; c++) tp[c + 1] += tp[c];
        std::vector<int32_t> tr(nnzA);
        {
            std::vector<int64_t> fill(tp.begin(), tp.end() - 1);
            for (int32_t r = 0; r < N; r++)
                for (int64_t k = rp[r]; k < rp[r + 1]; k++) tr[fill[ci[k]]++] = r;   // ascending r per column
        }

        // symmetric pattern <=> CSR(A) == CSR(A^T) (both have ascending columns)
        const bool symmetric = rp == tp && ci == tr;
        lap(0);
        // ---- candidate edges (reference rule, cpp:75-103), streamed and pruned ------------------
        // pair (i, j>i) with s shared columns: h = nnz_i + nnz_j - 2s;
        //   j -> i admitted iff h < nnz_i - alpha  <=>  2s > nnz_j + alpha
        //   i -> j admitted iff h < nnz_j - alpha  <=>  2s > nnz_i + alpha
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
                    const int32_t ni = nnz[i];
                    o.push_back({N, i, ni});
                    touched.clear();
                    for (int64_t k = rp[i]; k < rp[i + 1]; k++) {
                        const int32_t c = ci[k];
                        const int32_t* lo = tr.data() + tp[c];
                        const int32_t* hi = tr.data() + tp[c + 1];
                        for (const int32_t* q = std::upper_bound(lo, hi, i); q < hi; ++q) {
                            const int32_t j = *q;
                            if (cnt[j]++ == 0) touched.push_back(j);
                        }
                    }
                    adm.clear();
                    for (int32_t j : touched) {
                        const int32_t s = cnt[j];
                        cnt[j] = 0;
                        if (2 * s > std::min(ni, nnz[j]) + alpha) adm.push_back({j, s});
                    }
                    std::sort(adm.begin(), adm.end());
                    for (auto& js : adm) {
                        const int32_t j = js.first, nj = nnz[j];
                        const int32_t h = ni + nj - 2 * js.second;
                        if (h < ni - alpha) o.push_back({j, i, h});
                        if (h < nj - alpha) o.push_back({i, j, h});
                    }
                }
            }
        }
        std::vector<CandEdge> cand;
        {
            size_t tot = 0;
            for (auto& o : chunk_out) tot += o.size();
            cand.reserve(tot);
            for (auto& o : chunk_out) { cand.insert(cand.end(), o.begin(), o.end()); std::vector<CandEdge>().swap(o); }
        }
        if (cand.size() >= (size_t)INT32_MAX) return CBM_ERR_SHAPE;

        lap(1);
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
        std::vector<int32_t> mst_row(N + 2, 0), mst_col(N);
        for (int32_t v = 0; v < N; v++) mst_row[par[v] + 1]++;
        for (int32_t u = 0; u <= N; u++) mst_row[u + 1] += mst_row[u];
        {
            std::vector<int32_t> fill(mst_row.begin(), mst_row.end() - 1);
            for (int32_t v = 0; v < N; v++) mst_col[fill[par[v]]++] = v;
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
        if (run != weight) return CBM_ERR_INTERNAL;      // nnz(delta) must equal the arborescence weight
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
    } catch (const std::bad_alloc&) {
        cbm_format_free(out);
        return CBM_ERR_ALLOC;
    }
}

}  // extern "C"
