/*
 * CPU oracle for the CBM (compressed binary matrix) multiply -- TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference's CPU path so that the HIP
 * kernels can be checked against it.  Nothing in the shipped package may link, load or call
 * it; only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py do.
 *
 * Reference lines each function follows (all under /root/reference/cbm/cbm_extensions.cpp):
 *   oracle_build            :8-326 (plain builder), :328-644 (normalised builder; same tree,
 *                           delta values scaled by col_mul[col], :504-585)
 *   oracle_csr_spmm         :790-843 / :1707-1755  (mkl_sparse_s_mm, row-major, alpha=1, beta=0)
 *   oracle_update_plain     :713-738 (seq) and :1166-1218 (omp, schedule(dynamic,50))
 *   oracle_update_fused     :908-995 (seq) and :1285-1373 (omp)
 *
 * Third-party pieces absent from /root/reference and what stands in for them here:
 *   arbok::TarjanPQ (un-vendored submodule, unpinned)  -> oracle_msa(): Chu-Liu/Edmonds by
 *       repeated cycle contraction with edge recovery.  Any minimum arborescence has the same
 *       weight; WHICH one arbok returns among ties is "parity unpinned".
 *   Intel MKL mkl_sparse_syrk                          -> sparse-accumulator row intersections.
 *   Intel MKL mkl_sparse_s_mm                          -> in-order fp32 FMA accumulation per
 *       output element; MKL's own summation order is opaque, so agreement with the reference
 *       is to tolerance (1e-4), the level the reference's own tests pin.
 *
 * What pins this oracle (tests/test_oracle.py): brute-force candidate rule on dense A*A^T,
 * arborescence weight against networkx and exhaustive enumeration, set reconstruction of every
 * row (the reference's check_format, cbm/cbm.py:69-115), dense fp64 A@X closed forms with
 * integer features (bit-exact), flat-tree / identical-row / clique special cases.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_OK 0
#define ORACLE_ERR_ALLOC 2
#define ORACLE_ERR_ARG 3

static int cmp_i32(const void* a, const void* b) {
    int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
    return (x > y) - (x < y);
}

void oracle_free(void* p) { free(p); }

/* ------------------------------------------------------------------------------------------
 * Minimum spanning arborescence rooted at `root` on n nodes and m edges (eu -> ev, weight ew).
 * Every node must be reachable from the root (the CBM distance graph has a root edge to every
 * row).  chosen[v] receives the index of the edge entering v (chosen[root] = -1).
 * Chu-Liu/Edmonds: pick the cheapest in-edge of every node, contract the cycles, reduce the
 * weights of edges entering a contracted node by the in-edge they would replace, repeat; the
 * choice is unwound afterwards through (add, del) records.
 * ---------------------------------------------------------------------------------------- */
int oracle_msa(int32_t n, int64_t m, const int32_t* eu, const int32_t* ev, const int32_t* ew,
               int32_t root, int64_t* chosen, int64_t* total_weight) {
    int64_t cap = m * 2 + 16, tot = m, cur_m = m;
    int32_t *cu = malloc(sizeof(int32_t) * (size_t)(m + 1)), *cv = malloc(sizeof(int32_t) * (size_t)(m + 1));
    int64_t *cw = malloc(sizeof(int64_t) * (size_t)(m + 1)), *cid = malloc(sizeof(int64_t) * (size_t)(m + 1));
    int64_t *add = malloc(sizeof(int64_t) * (size_t)cap), *del = malloc(sizeof(int64_t) * (size_t)cap);
    int32_t* used = calloc((size_t)cap, sizeof(int32_t));
    int64_t *in_id = malloc(sizeof(int64_t) * (size_t)n), *in_w = malloc(sizeof(int64_t) * (size_t)n);
    int32_t *in_u = malloc(sizeof(int32_t) * (size_t)n), *comp = malloc(sizeof(int32_t) * (size_t)n);
    int32_t* mark = malloc(sizeof(int32_t) * (size_t)n);
    if (!cu || !cv || !cw || !cid || !add || !del || !used || !in_id || !in_w || !in_u || !comp || !mark)
        return ORACLE_ERR_ALLOC;
    for (int64_t e = 0; e < m; e++) { cu[e] = eu[e]; cv[e] = ev[e]; cw[e] = ew[e]; cid[e] = e; add[e] = del[e] = -1; }
    int32_t cur_n = n, cur_root = root;
    for (;;) {
        for (int32_t v = 0; v < cur_n; v++) { in_id[v] = -1; in_w[v] = 0; in_u[v] = -1; }
        for (int64_t e = 0; e < cur_m; e++) {
            int32_t u = cu[e], v = cv[e];
            if (u == v || v == cur_root) continue;
            if (in_id[v] < 0 || cw[e] < in_w[v]) { in_id[v] = cid[e]; in_w[v] = cw[e]; in_u[v] = u; }
        }
        for (int32_t v = 0; v < cur_n; v++) {
            if (v == cur_root) continue;
            if (in_id[v] < 0) return ORACLE_ERR_ARG;           /* unreachable node */
            used[in_id[v]]++;
        }
        /* find cycles of the in-edge functional graph */
        int32_t n_comp = 0, cycles = 0;
        for (int32_t v = 0; v < cur_n; v++) { comp[v] = -1; mark[v] = -1; }
        for (int32_t s = 0; s < cur_n; s++) {
            int32_t v = s;
            while (v != cur_root && mark[v] < 0 && comp[v] < 0) { mark[v] = s; v = in_u[v]; }
            if (v != cur_root && comp[v] < 0 && mark[v] == s) {  /* closed a new cycle at v */
                int32_t c = n_comp++;
                cycles++;
                int32_t x = v;
                do { comp[x] = c; x = in_u[x]; } while (x != v);
            }
        }
        if (cycles == 0) break;
        for (int32_t v = 0; v < cur_n; v++) if (comp[v] < 0) comp[v] = n_comp++;
        int64_t out = 0;
        for (int64_t e = 0; e < cur_m; e++) {
            int32_t u = cu[e], v = cv[e];
            int32_t nu = comp[u], nv = comp[v];
            if (nu == nv || v == cur_root) continue;
            if (tot >= cap) {
                int64_t ncap = cap * 2;
                add = realloc(add, sizeof(int64_t) * (size_t)ncap);
                del = realloc(del, sizeof(int64_t) * (size_t)ncap);
                used = realloc(used, sizeof(int32_t) * (size_t)ncap);
                if (!add || !del || !used) return ORACLE_ERR_ALLOC;
                memset(used + cap, 0, sizeof(int32_t) * (size_t)(ncap - cap));
                cap = ncap;
            }
            add[tot] = cid[e]; del[tot] = in_id[v];
            cu[out] = nu; cv[out] = nv; cw[out] = cw[e] - in_w[v]; cid[out] = tot;
            tot++; out++;
        }
        cur_m = out; cur_root = comp[cur_root]; cur_n = n_comp;
    }
    for (int64_t i = tot - 1; i >= m; i--)
        if (used[i] > 0) { used[del[i]] -= used[i]; used[add[i]] += used[i]; }
    int64_t w = 0;
    for (int32_t v = 0; v < n; v++) chosen[v] = -1;
    for (int64_t e = 0; e < m; e++)
        if (used[e] > 0) { if (chosen[ev[e]] >= 0) return ORACLE_ERR_ARG; chosen[ev[e]] = e; w += ew[e]; }
    for (int32_t v = 0; v < n; v++) if (v != root && chosen[v] < 0) return ORACLE_ERR_ARG;
    *total_weight = w;
    free(cu); free(cv); free(cw); free(cid); free(add); free(del); free(used);
    free(in_id); free(in_w); free(in_u); free(comp); free(mark);
    return ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------
 * Candidate edges of the distance graph, cpp:71-103.  Emission order is the reference's: for
 * row i ascending: (root -> i, nnz_i); then for j > i ascending with |row_i ^ row_j| > 0:
 * h = nnz_i + nnz_j - 2|row_i ^ row_j|;  (j -> i, h) if h < nnz_i - alpha;  (i -> j, h) if
 * h < nnz_j - alpha.  rp/ci is CSR(A) with sorted unique columns.
 * ---------------------------------------------------------------------------------------- */
int oracle_candidates(int32_t N, const int64_t* rp, const int32_t* ci, int32_t alpha,
                      int32_t** out_u, int32_t** out_v, int32_t** out_w, int64_t* out_m) {
    int64_t E = rp[N];
    /* transpose (column -> rows containing it) */
    int64_t* tp = calloc((size_t)N + 2, sizeof(int64_t));
    int32_t* tr = malloc(sizeof(int32_t) * (size_t)(E + 1));
    int32_t* cnt = calloc((size_t)N + 1, sizeof(int32_t));
    int32_t* touched = malloc(sizeof(int32_t) * (size_t)(N + 1));
    if (!tp || !tr || !cnt || !touched) return ORACLE_ERR_ALLOC;
    for (int64_t k = 0; k < E; k++) tp[ci[k] + 1]++;
    for (int32_t c = 0; c < N; c++) tp[c + 1] += tp[c];
    {
        int64_t* fill = malloc(sizeof(int64_t) * (size_t)(N + 1));
        if (!fill) return ORACLE_ERR_ALLOC;
        memcpy(fill, tp, sizeof(int64_t) * (size_t)(N + 1));
        for (int32_t r = 0; r < N; r++)
            for (int64_t k = rp[r]; k < rp[r + 1]; k++) tr[fill[ci[k]]++] = r;
        free(fill);
    }
    int64_t cap = (int64_t)N * 4 + 64, m = 0;
    int32_t *gu = malloc(sizeof(int32_t) * (size_t)cap), *gv = malloc(sizeof(int32_t) * (size_t)cap),
            *gw = malloc(sizeof(int32_t) * (size_t)cap);
    if (!gu || !gv || !gw) return ORACLE_ERR_ALLOC;
#define PUSH(U, V, W)                                                                 \
    do {                                                                              \
        if (m >= cap) {                                                               \
            cap *= 2;                                                                 \
            gu = realloc(gu, sizeof(int32_t) * (size_t)cap);                          \
            gv = realloc(gv, sizeof(int32_t) * (size_t)cap);                          \
            gw = realloc(gw, sizeof(int32_t) * (size_t)cap);                          \
            if (!gu || !gv || !gw) return ORACLE_ERR_ALLOC;                           \
        }                                                                             \
        gu[m] = (U); gv[m] = (V); gw[m] = (W); m++;                                   \
    } while (0)
    for (int32_t i = 0; i < N; i++) {
        int32_t nnz_i = (int32_t)(rp[i + 1] - rp[i]);
        PUSH(N, i, nnz_i);
        int32_t nt = 0;
        for (int64_t k = rp[i]; k < rp[i + 1]; k++) {
            int32_t c = ci[k];
            for (int64_t q = tp[c]; q < tp[c + 1]; q++) {
                int32_t j = tr[q];
                if (j <= i) continue;
                if (cnt[j]++ == 0) touched[nt++] = j;
            }
        }
        qsort(touched, (size_t)nt, sizeof(int32_t), cmp_i32);
        for (int32_t t = 0; t < nt; t++) {
            int32_t j = touched[t];
            int32_t s = cnt[j];
            cnt[j] = 0;
            int32_t nnz_j = (int32_t)(rp[j + 1] - rp[j]);
            int32_t h = nnz_i + nnz_j - 2 * s;
            if (h < nnz_i - alpha) PUSH(j, i, h);
            if (h < nnz_j - alpha) PUSH(i, j, h);
        }
    }
#undef PUSH
    free(tp); free(tr); free(cnt); free(touched);
    *out_u = gu; *out_v = gv; *out_w = gw; *out_m = m;
    return ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------
 * Full builder, cpp:8-326.  Input: COO (row, col) of a 0/1 matrix, any order, duplicates are
 * merged.  Output (malloc'd, release with oracle_free):
 *   mst_row[N+2], mst_col[N]  tree in CSR form, row N = the virtual root   (cpp:274-286)
 *   d_row, d_col, d_sign[nnz] delta entries in the reference's emission order (BFS from the
 *                             root, per row a sorted two-pointer merge, cpp:173-270)
 *   parent[N]                 parent of every row (N = virtual root)
 * Children of a node are visited in ascending id (the reference's order is whatever arbok's
 * reconstruct() yields: unpinned).
 * ---------------------------------------------------------------------------------------- */
int oracle_build(const int32_t* row, const int32_t* col, int64_t E, int32_t N, int32_t alpha,
                 int32_t** mst_row_o, int32_t** mst_col_o, int32_t** d_row_o, int32_t** d_col_o,
                 int8_t** d_sign_o, int64_t* nnz_delta_o, int32_t** parent_o,
                 int64_t* n_candidates_o, int64_t* msa_weight_o) {
    if (N <= 0 || E < 0) return ORACLE_ERR_ARG;
    /* COO -> CSR with sorted, unique columns (cpp:15-43) */
    int64_t* rp = calloc((size_t)N + 2, sizeof(int64_t));
    int32_t* ci = malloc(sizeof(int32_t) * (size_t)(E + 1));
    if (!rp || !ci) return ORACLE_ERR_ALLOC;
    for (int64_t k = 0; k < E; k++) {
        if (row[k] < 0 || row[k] >= N || col[k] < 0 || col[k] >= N) return ORACLE_ERR_ARG;
        rp[row[k] + 1]++;
    }
    for (int32_t r = 0; r < N; r++) rp[r + 1] += rp[r];
    {
        int64_t* fill = malloc(sizeof(int64_t) * (size_t)(N + 1));
        if (!fill) return ORACLE_ERR_ALLOC;
        memcpy(fill, rp, sizeof(int64_t) * (size_t)(N + 1));
        for (int64_t k = 0; k < E; k++) ci[fill[row[k]]++] = col[k];
        free(fill);
        int64_t w = 0;
        int64_t* nrp = calloc((size_t)N + 2, sizeof(int64_t));
        if (!nrp) return ORACLE_ERR_ALLOC;
        for (int32_t r = 0; r < N; r++) {
            int64_t b = rp[r], e = rp[r + 1];
            qsort(ci + b, (size_t)(e - b), sizeof(int32_t), cmp_i32);
            nrp[r] = w;
            for (int64_t k = b; k < e; k++)
                if (k == b || ci[k] != ci[k - 1]) ci[w++] = ci[k];
        }
        nrp[N] = w;
        free(rp);
        rp = nrp;
    }
    int32_t *gu, *gv, *gw;
    int64_t m;
    int rc = oracle_candidates(N, rp, ci, alpha, &gu, &gv, &gw, &m);
    if (rc) return rc;
    int64_t* chosen = malloc(sizeof(int64_t) * (size_t)(N + 1));
    int64_t weight = 0;
    if (!chosen) return ORACLE_ERR_ALLOC;
    rc = oracle_msa(N + 1, m, gu, gv, gw, N, chosen, &weight);
    if (rc) return rc;
    int32_t* parent = malloc(sizeof(int32_t) * (size_t)N);
    int32_t* mst_row = calloc((size_t)N + 2, sizeof(int32_t));
    int32_t* mst_col = malloc(sizeof(int32_t) * (size_t)N);
    if (!parent || !mst_row || !mst_col) return ORACLE_ERR_ALLOC;
    for (int32_t v = 0; v < N; v++) { parent[v] = gu[chosen[v]]; mst_row[parent[v] + 1]++; }
    for (int32_t u = 0; u <= N; u++) mst_row[u + 1] += mst_row[u];
    {
        int32_t* fill = malloc(sizeof(int32_t) * (size_t)(N + 1));
        if (!fill) return ORACLE_ERR_ALLOC;
        memcpy(fill, mst_row, sizeof(int32_t) * (size_t)(N + 1));
        for (int32_t v = 0; v < N; v++) mst_col[fill[parent[v]]++] = v;   /* ascending v per parent */
        free(fill);
    }
    /* BFS from the root, emitting deltas on first visit (cpp:173-270) */
    int64_t dcap = weight + 16, nd = 0;
    int32_t *d_row = malloc(sizeof(int32_t) * (size_t)dcap), *d_col = malloc(sizeof(int32_t) * (size_t)dcap);
    int8_t* d_sign = malloc((size_t)dcap);
    int32_t* fifo = malloc(sizeof(int32_t) * (size_t)(N + 1));
    if (!d_row || !d_col || !d_sign || !fifo) return ORACLE_ERR_ALLOC;
    int32_t head = 0, tail = 0, visited = 0;
    fifo[tail++] = N;
    while (head < tail) {
        int32_t u = fifo[head++];
        for (int32_t q = mst_row[u]; q < mst_row[u + 1]; q++) {
            int32_t v = mst_col[q];
            fifo[tail++] = v;
            visited++;
            int64_t vp = rp[v], ve = rp[v + 1];
            if (u == N) {
                for (; vp < ve; vp++) { d_row[nd] = v; d_col[nd] = ci[vp]; d_sign[nd] = 1; nd++; }
            } else {
                int64_t up = rp[u], ue = rp[u + 1];
                while (up < ue && vp < ve) {
                    if (ci[up] == ci[vp]) { up++; vp++; }
                    else if (ci[up] > ci[vp]) { d_row[nd] = v; d_col[nd] = ci[vp]; d_sign[nd] = 1; nd++; vp++; }
                    else { d_row[nd] = v; d_col[nd] = ci[up]; d_sign[nd] = -1; nd++; up++; }
                }
                for (; up < ue; up++) { d_row[nd] = v; d_col[nd] = ci[up]; d_sign[nd] = -1; nd++; }
                for (; vp < ve; vp++) { d_row[nd] = v; d_col[nd] = ci[vp]; d_sign[nd] = 1; nd++; }
            }
            if (nd > weight) return ORACLE_ERR_ARG;   /* delta count must equal the MSA weight */
        }
    }
    if (visited != N || nd != weight) return ORACLE_ERR_ARG;
    free(fifo); free(chosen); free(gu); free(gv); free(gw); free(rp); free(ci);
    *mst_row_o = mst_row; *mst_col_o = mst_col; *d_row_o = d_row; *d_col_o = d_col; *d_sign_o = d_sign;
    *nnz_delta_o = nd; *parent_o = parent; *n_candidates_o = m; *msa_weight_o = weight;
    return ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------
 * Y = A * X, 4-array CSR, row-major X[N x d], beta = 0 (cpp:790-843, :1707-1755).
 * ---------------------------------------------------------------------------------------- */
void oracle_csr_spmm(const int32_t* row_b, const int32_t* row_e, const int32_t* col, const float* val,
                     const float* X, float* Y, int32_t N, int32_t d, int32_t threads) {
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 64) num_threads(threads > 0 ? threads : 1)
#endif
    for (int32_t r = 0; r < N; r++) {
        float* y = Y + (size_t)r * d;
        for (int32_t j = 0; j < d; j++) y[j] = 0.0f;
        for (int32_t k = row_b[r]; k < row_e[r]; k++) {
            const float a = val ? val[k] : 1.0f;
            const float* x = X + (size_t)col[k] * d;
            for (int32_t j = 0; j < d; j++) y[j] = fmaf(a, x[j], y[j]);
        }
    }
}

/* Same product with the summation order of a SIMD kernel that deals the entries of a row to
 * `groups` lanes round-robin: partial sum g takes entries k = g (mod groups) in order (FMA), and
 * the partial sums are combined by a butterfly (xor 1, 2, 4, ...), i.e. a balanced binary tree.
 * groups must be a power of two <= 64; groups == 1 is oracle_csr_spmm.  MKL's own order inside
 * mkl_sparse_s_mm is not documented, so this is as valid a restatement of cpp:1149-1159 as the
 * in-order one; it exists so that GPU results can be compared bit for bit. */
void oracle_csr_spmm_grouped(const int32_t* row_b, const int32_t* row_e, const int32_t* col, const float* val,
                             const float* X, float* Y, int32_t N, int32_t d, int32_t groups, int32_t threads) {
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 64) num_threads(threads > 0 ? threads : 1)
#endif
    for (int32_t r = 0; r < N; r++) {
        float* y = Y + (size_t)r * d;
        for (int32_t j = 0; j < d; j++) {
            float part[64];
            for (int32_t g = 0; g < groups; g++) part[g] = 0.0f;
            for (int32_t k = row_b[r]; k < row_e[r]; k++) {
                const int32_t g = (k - row_b[r]) % groups;
                part[g] = fmaf(val ? val[k] : 1.0f, X[(size_t)col[k] * d + j], part[g]);
            }
            for (int32_t off = 1; off < groups; off <<= 1) {
                float next[64];
                for (int32_t g = 0; g < groups; g++) next[g] = part[g] + part[g ^ off];
                for (int32_t g = 0; g < groups; g++) part[g] = next[g];
            }
            y[j] = part[0];
        }
    }
}

/* Tree walk, plain: Y[v,:] += Y[parent(v),:] top-down (cpp:713-738; omp :1166-1218).
 * mst_row has N+2 entries; the root's children are mst_col[mst_row[N] .. mst_row[N+1]). */
void oracle_update_plain(const int32_t* mst_row, const int32_t* mst_col, float* Y, int32_t N, int32_t d,
                         int32_t threads) {
    const int32_t jb = mst_row[N], je = mst_row[N + 1];
#ifdef _OPENMP
#pragma omp parallel num_threads(threads > 0 ? threads : 1)
#endif
    {
        int32_t* lifo = malloc(sizeof(int32_t) * (size_t)(N + 1));
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 50)
#endif
        for (int32_t j = jb; j < je; j++) {
            int32_t top = 0;
            lifo[top++] = mst_col[j];
            while (top > 0) {
                int32_t u = lifo[--top];
                for (int32_t q = mst_row[u]; q < mst_row[u + 1]; q++) {
                    int32_t v = mst_col[q];
                    const float* x = Y + (size_t)u * d;
                    float* y = Y + (size_t)v * d;
                    for (int32_t i = 0; i < d; i++) y[i] += x[i];
                    lifo[top++] = v;
                }
            }
        }
        free(lifo);
    }
}

/* Tree walk, GCN-normalised: root child Y[r] *= m[r] (cpp:910-940); tree edge u -> v:
 * Y[v] = fma(Y[u], 1/m[u], Y[v]) * m[v] in the 16- and 8-wide vector body (cpp:966-986), and
 * (Y[v] + Y[u]/m[u]) * m[v] in the scalar tail of d mod 8 elements (cpp:988-990). */
void oracle_update_fused(const int32_t* mst_row, const int32_t* mst_col, const float* m, float* Y,
                         int32_t N, int32_t d, int32_t threads) {
    const int32_t jb = mst_row[N], je = mst_row[N + 1];
    const int32_t dv = d - (d % 8);
#ifdef _OPENMP
#pragma omp parallel num_threads(threads > 0 ? threads : 1)
#endif
    {
        int32_t* lifo = malloc(sizeof(int32_t) * (size_t)(N + 1));
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 50)
#endif
        for (int32_t j = jb; j < je; j++) {
            const int32_t r = mst_col[j];
            float* yr = Y + (size_t)r * d;
            const float r_scale = m[r];
            for (int32_t i = 0; i < d; i++) yr[i] *= r_scale;
            int32_t top = 0;
            lifo[top++] = r;
            while (top > 0) {
                int32_t u = lifo[--top];
                const float u_scale = m[u];
                const float u_inv = 1 / u_scale;
                for (int32_t q = mst_row[u]; q < mst_row[u + 1]; q++) {
                    int32_t v = mst_col[q];
                    const float v_scale = m[v];
                    const float* x = Y + (size_t)u * d;
                    float* y = Y + (size_t)v * d;
                    int32_t i = 0;
                    for (; i < dv; i++) y[i] = fmaf(x[i], u_inv, y[i]) * v_scale;
                    for (; i < d; i++) y[i] = (y[i] + (x[i] / u_scale)) * v_scale;
                    lifo[top++] = v;
                }
            }
        }
        free(lifo);
    }
}

int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
