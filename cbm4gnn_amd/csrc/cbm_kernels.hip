// HIP kernels (gfx950 / CDNA4) and C-ABI launchers of the CBM multiply.
//
// Bandwidth-bound gather / stream kernels, 64-wide wavefronts, no MFMA, no atomics:
//   (1)  spmm_slab_per_xcd    delta SpMM  Z = D * diag(m) * X  with the feature dimension cut into
//                             128-byte slabs (256-byte on the row-major path of wide d): one slab per
//                             XCD (so an XCD's L2 only ever sees its slab of X), persistent waves
//                             walking a longest-first row schedule.  Long rows: one row per wave, 8
//                             lanes per delta entry, 64 entries in flight.  Short rows (a batched
//                             schedule): 8 rows per wave, one lane group each, entries in order.  Any
//                             width when the caller brings a workspace for the slab-major copy of X
//                             (relayout_slabs).
//        spmm_tiled_local     the same product for matrices whose entries cluster: tiles of the copy
//                             staged in LDS, one row per lane group, the scattered rest from the copy
//                             in global memory in the same launch.
//        spmm_wave_per_row    the same product without a workspace for widths that are not a
//                             multiple of 32: one wave per row, lanes span the feature columns,
//                             packed indices broadcast with v_readlane so X-row addresses are scalar.
//   (2)  tree propagation  Y[v] (+)= Y[parent(v)]:
//        propagate_level / propagate_narrow_levels / propagate_chain / scale_level0
//                             level-synchronously over a host-computed (level, id) ordering: one
//                             launch per wide level, one single-workgroup launch per run of narrow
//                             levels, one register-carried launch per chain of single-row levels;
//        propagate_subtrees   every subtree below a level in ONE launch: a wave walks a host-made
//                             depth-first sequence, parent values in a register and LDS slots;
//        spmm_update_subtrees the same walk with every row's delta entries summed on the way (deep trees,
//                             short delta rows): SpMM and walk in one launch, no SpMM result in memory;
//        propagate_paths / spmm_update_paths_wave_per_row
//                             shallow trees: every row sums down its own ancestor path (one launch).
// The SpMM instantiations with PACKED = false are the plain CSR baseline.
//
// What each launcher replaces in the reference is stated in include/cbm_hip.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <type_traits>

#include "../../include/cbm_hip.h"

namespace {

// Tunables (overridable with -D for sweeps; the defaults are what measurements on MI355X chose:
// 2, 8 or 16 waves per workgroup, 4 or 16 loads in flight and no XCD remap were all within +-3 %
// or slower on the 100k-node power-law workload).
#ifndef CBM_WAVES_PER_BLOCK
#define CBM_WAVES_PER_BLOCK 4
#endif
#ifndef CBM_UNROLL_CH1
#define CBM_UNROLL_CH1 8
#endif
#ifndef CBM_SLAB_ROUNDS
#define CBM_SLAB_ROUNDS 8                  // load instructions in flight per wave in the slab kernel
#endif
#ifndef CBM_TILED_VECS
#define CBM_TILED_VECS 6                   // 16-byte index vectors requested together per row in the tiled kernel
#endif
#ifndef CBM_TILED_REMOTE_U8
#define CBM_TILED_REMOTE_U8 6              // remote entries per row in flight in the tiled kernel, 128-byte slabs (2 rows per lane):
                                           // 8 need 24 registers more than a 1024-thread workgroup has (spilled: 1.62 ms on the
                                           // 233k-row community graph at d = 128), 7: 1.58, 6: 1.57 with none spilled, 5: 1.58
#endif
#ifndef CBM_TILED_REMOTE_U4
#define CBM_TILED_REMOTE_U4 8              // the same for the 64-byte half slab (1 row per lane)
#endif
#ifndef CBM_XCD_REMAP
#define CBM_XCD_REMAP 1
#endif

constexpr int kWave = 64;
constexpr int kWavesPerBlock = CBM_WAVES_PER_BLOCK;   // SpMM / wide-level propagate
constexpr int kMaxPathLevels = CBM_PATH_MAX_LEVELS;   // deepest tree the one-launch walks take
constexpr int kNarrowWaves = 16;           // narrow-level propagate: one 1024-thread workgroup
constexpr int kNarrowWidth = 64;           // a level with at most this many rows is "narrow"
constexpr int kXcds = 8;                   // MI355X: 8 XCDs, workgroups are dealt round-robin

// Workgroup ids are dealt to the 8 XCDs round-robin; give every XCD a contiguous range of
// logical blocks so that neighbouring rows (which share columns in clustered graphs) meet in
// the same L2.
__device__ __forceinline__ int xcd_contiguous_block(int bid, int nb) {
    if (!CBM_XCD_REMAP) return bid;
    const int q = nb / kXcds, r = nb % kXcds;
    const int x = bid % kXcds;
    return x * q + (x < r ? x : r) + bid / kXcds;
}

template <int VEC>
__device__ __forceinline__ void load_vec(const float* __restrict__ p, float (&v)[VEC]) {
    if constexpr (VEC == 4) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else if constexpr (VEC == 2) {
        const float2 t = *reinterpret_cast<const float2*>(p);
        v[0] = t.x; v[1] = t.y;
    } else {
        v[0] = *p;
    }
}

template <int VEC>
__device__ __forceinline__ void store_vec(float* __restrict__ p, const float (&v)[VEC]) {
    if constexpr (VEC == 4) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else if constexpr (VEC == 2) {
        *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
    } else {
        *p = v[0];
    }
}

__device__ __forceinline__ int bcast_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float bcast_f(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// ---------------------------------------------------------------------------------------------
// (1) SpMM, one wavefront per row.
//   PACKED: idx = col | sign<<31, coefficient = +-1 or +-m[col]
//   !PACKED: idx = col (int32), coefficient = val[k] or 1
//   VEC floats per lane per chunk, CH chunks of 64*VEC columns per wave; grid.y tiles wider d.
//   FULL: d is an exact multiple of the tile, no column guards.
// ---------------------------------------------------------------------------------------------
template <int VEC, int CH, bool PACKED, bool FULL>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void spmm_wave_per_row(
    const int32_t* __restrict__ rowptr, const uint32_t* __restrict__ idx, const float* __restrict__ val,
    const float* __restrict__ m, const int32_t* __restrict__ parent, const int4* __restrict__ sched,
    const float* __restrict__ X, float* __restrict__ Z, int n, int d, int64_t ldx, int64_t ldz, int relu) {
    constexpr int U = (CH == 1) ? CBM_UNROLL_CH1 : (CH == 2 ? CBM_UNROLL_CH1 / 2 : CBM_UNROLL_CH1 / 4);   // X-row loads in flight per wave
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    int row = xcd_contiguous_block(blockIdx.x, gridDim.x) * kWavesPerBlock + wave;
    if (row >= n) return;
    int start, end;
    float root_scale = 1.0f;                   // left scaling of root children, fetched up front
    if (sched) {
        const int4 r = sched[row];
        start = __builtin_amdgcn_readfirstlane(r.x);
        end = __builtin_amdgcn_readfirstlane(r.y);
        row = __builtin_amdgcn_readfirstlane(r.z);
        root_scale = __int_as_float(__builtin_amdgcn_readfirstlane(r.w));
    } else {
        row = __builtin_amdgcn_readfirstlane(row);
        start = __builtin_amdgcn_readfirstlane(rowptr[row]);
        end = __builtin_amdgcn_readfirstlane(rowptr[row + 1]);
        if constexpr (PACKED) {
            if (m && parent) {
                const int par = parent[row];
                const float mr = m[row];
                root_scale = par < 0 ? mr : 1.0f;
            }
        }
    }
    const int col0 = blockIdx.y * (kWave * VEC * CH) + lane * VEC;

    float acc[CH][VEC];
#pragma unroll
    for (int c = 0; c < CH; c++)
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[c][v] = 0.0f;

    // One coalesced load brings 64 packed indices into the wave and, in the same step, each lane
    // resolves the coefficient of its entry (sign bit, m[col] gather, or the streamed CSR value);
    // entry k is then broadcast with v_readlane into scalar registers, so the row address of X
    // is wave-uniform and the only per-entry vector memory traffic is the X row itself.
    // (Looking m[col] up per entry through the scalar cache instead measured 3% slower.)
    for (int base = start; base < end; base += kWave) {
        const int cnt = min(kWave, end - base);
        int my_col = 0;
        float my_cf = 0.0f;
        if (lane < cnt) {
            if constexpr (PACKED) {
                const uint32_t p = idx[base + lane];
                my_col = (int)(p & 0x7fffffffu);
                if (val) my_cf = val[base + lane];                     // streamed +-m[col]
                else {
                    const uint32_t mag = m ? __float_as_uint(m[my_col]) : 0x3f800000u;
                    my_cf = __uint_as_float(mag ^ (p & 0x80000000u));  // +-1 or +-m[col], exact
                }
            } else {
                my_col = (int)idx[base + lane];
                my_cf = val ? val[base + lane] : 1.0f;
            }
        }
        // U X-row loads in flight; in the last, partial group the surplus loads repeat the row of
        // the last entry with coefficient 0 (a branch around each load would serialise them)
        for (int k = 0; k < cnt; k += U) {
            float x[U][CH][VEC];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float* __restrict__ xr = X + (int64_t)bcast_i(my_col, min(k + u, cnt - 1)) * ldx + col0;
#pragma unroll
                for (int c = 0; c < CH; c++) {
                    if (FULL || col0 + c * kWave * VEC < d) load_vec<VEC>(xr + c * kWave * VEC, x[u][c]);
                    else
#pragma unroll
                        for (int v = 0; v < VEC; v++) x[u][c][v] = 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float f = k + u < cnt ? bcast_f(my_cf, min(k + u, cnt - 1)) : 0.0f;
#pragma unroll
                for (int c = 0; c < CH; c++)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[c][v] = fmaf(f, x[u][c][v], acc[c][v]);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < CH; c++)                   // 1.0f unless a child of the root (left scaling)
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            acc[c][v] *= root_scale;
            if (relu) acc[c][v] = acc[c][v] < 0.0f ? 0.0f : acc[c][v];      // keeps NaN, as torch.relu does
        }
    float* __restrict__ zr = Z + (int64_t)row * ldz + col0;
#pragma unroll
    for (int c = 0; c < CH; c++)
        if (FULL || col0 + c * kWave * VEC < d) store_vec<VEC>(zr + c * kWave * VEC, acc[c]);
}


// ---------------------------------------------------------------------------------------------
// (1a) The whole product in ONE launch, for small matrices with shallow, sparse trees: the
// wavefront of row v follows parent[] up to the child of the root above it, then computes the
// delta-row sum of every row on that path (exactly the loop of spmm_wave_per_row: entries strictly
// in order, coefficient +-1, +-m[col] or streamed) and combines them top-down with the
// arithmetic of propagate_row -- so Y[v] is bit for bit what spmm_wave_per_row followed by the
// level-by-level walk returns.  Ancestors' sums are recomputed by every descendant: sum over rows
// of the delta entries on their paths instead of nnz, which pays only where a launch costs more
// than the extra gathers (a 4,096-row graph: 17 -> 11 us).  The caller decides.
// ---------------------------------------------------------------------------------------------
template <int VEC, int CH, bool NORM, bool FULL>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void spmm_update_paths_wave_per_row(
    const int32_t* __restrict__ rowptr, const uint32_t* __restrict__ idx, const float* __restrict__ val,
    const float* __restrict__ m, const int32_t* __restrict__ parent, const float* __restrict__ X,
    float* __restrict__ Y, int n, int d, int dv, int64_t ldx, int64_t ldy, int relu) {
    constexpr int U = (CH == 1) ? CBM_UNROLL_CH1 : (CH == 2 ? CBM_UNROLL_CH1 / 2 : CBM_UNROLL_CH1 / 4);
    const int lane = threadIdx.x & (kWave - 1);
    const int v = __builtin_amdgcn_readfirstlane(blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6));
    if (v >= n) return;
    const int col0 = blockIdx.y * (kWave * VEC * CH) + lane * VEC;
    // lane t keeps the ancestor t steps above v (lane 0: v itself); k = steps to the child of the root
    int path = v, k = 0;
    for (int u = __builtin_amdgcn_readfirstlane(parent[v]); u >= 0 && k < kMaxPathLevels - 1;
         u = __builtin_amdgcn_readfirstlane(parent[u])) {
        k++;
        if (lane == k) path = u;
    }
    float my_m = 1.0f;
    if constexpr (NORM) if (lane <= k) my_m = m[path];
    float run[CH][VEC];
    float mu = 1.0f;
    for (int t = k; t >= 0; t--) {
        const int a = bcast_i(path, t);
        const int start = __builtin_amdgcn_readfirstlane(rowptr[a]);
        const int end = __builtin_amdgcn_readfirstlane(rowptr[a + 1]);
        float acc[CH][VEC];
#pragma unroll
        for (int c = 0; c < CH; c++)
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[c][e] = 0.0f;
        for (int base = start; base < end; base += kWave) {
            const int cnt = min(kWave, end - base);
            int my_col = 0;
            float my_cf = 0.0f;
            if (lane < cnt) {
                const uint32_t p = idx[base + lane];
                my_col = (int)(p & 0x7fffffffu);
                if (val) my_cf = val[base + lane];                     // streamed +-m[col]
                else {
                    const uint32_t mag = NORM ? __float_as_uint(m[my_col]) : 0x3f800000u;
                    my_cf = __uint_as_float(mag ^ (p & 0x80000000u));  // +-1 or +-m[col], exact
                }
            }
            for (int q = 0; q < cnt; q += U) {
                float x[U][CH][VEC];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const float* __restrict__ xr = X + (int64_t)bcast_i(my_col, min(q + u, cnt - 1)) * ldx + col0;
#pragma unroll
                    for (int c = 0; c < CH; c++) {
                        if (FULL || col0 + c * kWave * VEC < d) load_vec<VEC>(xr + c * kWave * VEC, x[u][c]);
                        else
#pragma unroll
                            for (int e = 0; e < VEC; e++) x[u][c][e] = 0.0f;
                    }
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const float f = q + u < cnt ? bcast_f(my_cf, min(q + u, cnt - 1)) : 0.0f;
#pragma unroll
                    for (int c = 0; c < CH; c++)
#pragma unroll
                        for (int e = 0; e < VEC; e++) acc[c][e] = fmaf(f, x[u][c][e], acc[c][e]);
                }
            }
        }
        const float mv = bcast_f(my_m, t);
        if (t == k) {                                      // the child of the root: its sum, scaled from the left
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int e = 0; e < VEC; e++) run[c][e] = NORM ? acc[c][e] * mv : acc[c][e];
        } else {
            const float inv_mu = 1.0f / mu;
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    if constexpr (NORM) {
                        const int j = col0 + c * kWave * VEC + e;
                        run[c][e] = (j < dv) ? fmaf(run[c][e], inv_mu, acc[c][e]) * mv : (acc[c][e] + run[c][e] / mu) * mv;
                    } else {
                        run[c][e] = acc[c][e] + run[c][e];
                    }
                }
        }
        mu = mv;
    }
    float* __restrict__ y = Y + (int64_t)v * ldy + col0;
#pragma unroll
    for (int c = 0; c < CH; c++)
        if (FULL || col0 + c * kWave * VEC < d) {
            if (relu) {
#pragma unroll
                for (int e = 0; e < VEC; e++) run[c][e] = run[c][e] < 0.0f ? 0.0f : run[c][e];   // keeps NaN
            }
            store_vec<VEC>(y + c * kWave * VEC, run[c]);
        }
}

// ---------------------------------------------------------------------------------------------
// (1b) SpMM with the feature dimension split into slabs, one slab per XCD.
//
// X is N x d fp32.  A workgroup on XCD x only ever touches the columns of its slab s (LPE float4
// per row: 128 B for LPE = 8, 256 B for LPE = 16) of X and Z, so the working set each XCD's 4 MB
// L2 sees is N x slab bytes instead of all of X: rows of X that many delta rows share stay
// resident.  Inside a wave, LPE lanes serve one delta entry and the 64 / LPE lane groups serve
// that many consecutive entries of the same row at once; each group keeps its own partial sum
// (entries k = g mod (64 / LPE), in order) and the partial sums are added by a xor-shuffle tree
// at the end of the row.  The price: index (and coefficient) arrays are streamed once per slab.
// Where an entry's coefficient comes from is a template parameter, so that the gather rounds hold
// no branch at all (with run-time tests of `val` and `m` between the loads of a round the plain
// +-1 variant ran latency-bound: 6.2 ms at 8 wavefronts per SIMD, 9.1 ms at 4, on a matrix the
// streamed variant multiplies in 5.9 ms):
//   kCoefStream: val[k] streamed (the CSR values, or +-m[col] precomputed by expand_coef)
//   kCoefSign:   +-1 from bit 31 of the index (plain CSR columns have it clear: +1)
//   kCoefSignM:  +-m[col], m gathered per entry
// Bit 31 is masked off the column in every mode.  PACKED only names the instantiation the packed
// delta format runs on (kernel traces then tell CBM launches from CSR baseline launches) and
// enables the left scale read from m when no row schedule is given.
// ---------------------------------------------------------------------------------------------
constexpr int kCoefStream = 0, kCoefSign = 1, kCoefSignM = 2;

template <int LPE, bool PACKED, int COEF, int U>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void spmm_slab_per_xcd(
    const int32_t* __restrict__ rowptr, const int4* __restrict__ sched, const uint32_t* __restrict__ idx,
    const float* __restrict__ val, const float* __restrict__ m, const int32_t* __restrict__ parent,
    const float* __restrict__ X, float* __restrict__ Z, int n, int d, int vec_out, int n_slabs,
    int64_t x_slab_stride, int64_t x_row_stride, int64_t ldz, int relu, float* __restrict__ partials, int batched) {
    // batched: the schedule comes from cbm_schedule_rows_batched -- descriptor n is a trailer whose first word
    // says how many descriptors are walked one row per wavefront; the rows behind them are short and taken
    // kStep at a time, one per lane group (below).
    // n is the number of row descriptors (rows of the matrix, unless the schedule cuts long rows
    // into pieces: a descriptor whose row field has CBM_SCHED_PIECE set is a piece, and its sum goes
    // to slot (row field & ~CBM_SCHED_PIECE) of `partials`, n_slabs x 32 floats per slot, unscaled).
    // d is the true feature width: slabs may reach past it (odd widths are zero-padded in the
    // slab-major copy) and nothing is stored beyond column d; vec_out says that rows of Z are
    // float4-addressable.
    // X is addressed as X[slab * x_slab_stride + row * x_row_stride + column in slab]: the caller's
    // row-major matrix (slab stride = slab width, row stride = ldx) or the slab-major copy made by
    // relayout_slabs (slab stride = n * slab width, row stride = slab width).
    constexpr int kSlab = LPE * 4;                         // floats per slab
    constexpr int kStep = kWave / LPE;                     // entries per wave instruction
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane / LPE;                            // which entry of a step
    const int li = lane % LPE;                             // float4 position inside the slab
    // Persistent waves.  Workgroup b runs on XCD b % 8; G workgroups per XCD.
    //   n_slabs >= 8 (a multiple of 8): XCD x walks slabs x, x + 8, ... one after the other, its
    //     4 G waves sharing the rows of the current slab cyclically;
    //   n_slabs < 8 (a divisor of 8): the 8 / n_slabs XCDs of a slab share its rows cyclically.
    // Rows come in schedule order (longest first), so a cyclic deal gives every wave the same mix.
    const int xcd = blockIdx.x % kXcds;
    const int G = gridDim.x / kXcds;
    int first, stride, slab0, slab_step;
    {
        const int j = blockIdx.x / kXcds;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        if (n_slabs >= kXcds) {
            first = j * kWavesPerBlock + wave; stride = G * kWavesPerBlock; slab0 = xcd; slab_step = kXcds;
        } else {
            const int share = kXcds / n_slabs;
            first = ((xcd / n_slabs) * G + j) * kWavesPerBlock + wave; stride = share * G * kWavesPerBlock;
            slab0 = xcd % n_slabs; slab_step = n_slabs;      // a single slab for this XCD
        }
    }
    const int n_wide = batched ? __builtin_amdgcn_readfirstlane(sched[n].x) : n;
    for (int slab = slab0; slab < n_slabs; slab += slab_step) {
        const float* __restrict__ Xs = X + slab * x_slab_stride + li * 4;
        float* __restrict__ Zs = Z + slab * kSlab + li * 4;
        // row descriptor {start, end, row, bits(left scale)} fetched one row ahead of its use
        auto fetch = [&](int i) -> int4 {
            if (sched) return sched[i];
            int4 r;
            r.x = rowptr[i]; r.y = rowptr[i + 1]; r.z = i; r.w = 0x3f800000;
            if constexpr (PACKED) {
                if (m && parent) r.w = parent[i] < 0 ? __float_as_int(m[i]) : 0x3f800000;
            }
            return r;
        };
        int i = first;
        int4 nxt = make_int4(0, 0, 0, 0);
        if (i < n_wide) nxt = fetch(i);
        while (i < n_wide) {
            const int start = __builtin_amdgcn_readfirstlane(nxt.x);
            const int end = __builtin_amdgcn_readfirstlane(nxt.y);
            const int row = __builtin_amdgcn_readfirstlane(nxt.z);
            const float row_scale = __int_as_float(__builtin_amdgcn_readfirstlane(nxt.w));
            i += stride;
            if (i < n_wide) nxt = fetch(i);

            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            // One gather round = UU instructions of kStep entries each.  Every load of a round is
            // unconditional -- entries past the end of the row are clamped to its last entry and
            // get coefficient 0 -- so the X-row loads are all in flight together; a branch or an
            // exec mask around each load would serialise them.  Short remainders take a shorter
            // round instead of mostly clamped instructions.
            auto round = [&](auto uu_tag, int pos) {
                constexpr int UU = decltype(uu_tag)::value;
                uint32_t p[UU];
                float f[UU];
                float x[UU][4];
                // The round's entries come in with ONE coalesced load (lane l fetches entry pos + l,
                // clamped) and reach their lane group through the LDS crossbar.  UU per-group loads of
                // the same few addresses cost the texture addresser about half of what the X loads
                // cost: 3-15 % of the kernel time on the workloads measured.
                const int k = pos + lane;
                const int kc = min(k, end - 1);
                const uint32_t p_all = idx[kc];
                float f_all = 0.0f;
                if constexpr (COEF == kCoefStream) f_all = val[kc];
                if constexpr (COEF == kCoefStream) f_all = k < end ? f_all : 0.0f;
#pragma unroll
                for (int u = 0; u < UU; u++) {
                    p[u] = __shfl(p_all, u * kStep + sub, kWave);
                    if constexpr (COEF == kCoefStream) f[u] = __shfl(f_all, u * kStep + sub, kWave);
                }
#pragma unroll
                for (int u = 0; u < UU; u++) {
                    const uint32_t c = p[u] & 0x7fffffffu;
                    if constexpr (COEF != kCoefStream) {
                        const uint32_t mag = COEF == kCoefSignM ? __float_as_uint(m[c]) : 0x3f800000u;
                        f[u] = pos + u * kStep + sub < end ? __uint_as_float(mag ^ (p[u] & 0x80000000u)) : 0.0f;
                    }
                    load_vec<4>(Xs + (int64_t)c * x_row_stride, x[u]);
                }
#pragma unroll
                for (int u = 0; u < UU; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[e] = fmaf(f[u], x[u][e], acc[e]);
            };
            int pos = start;
            while (pos < end) {
                const int rem = end - pos;
                if (rem > (U / 2) * kStep) { round(std::integral_constant<int, U>{}, pos); pos += U * kStep; }
                else if (rem > (U / 4) * kStep) { round(std::integral_constant<int, U / 2>{}, pos); pos += (U / 2) * kStep; }
                else if (rem > kStep) { round(std::integral_constant<int, U / 4>{}, pos); pos += (U / 4) * kStep; }
                else { round(std::integral_constant<int, 1>{}, pos); pos += kStep; }
            }
#pragma unroll
            for (int off = LPE; off < kWave; off <<= 1)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] += __shfl_xor(acc[e], off, kWave);
            if (sub == 0 && (row & CBM_SCHED_PIECE)) {                  // a piece of a cut row: raw sum to its slot
                store_vec<4>(partials + ((int64_t)(row & ~CBM_SCHED_PIECE) * n_slabs + slab) * kSlab + li * 4, acc);
            } else if (sub == 0) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc[e] *= row_scale;                              // 1.0f unless a child of the root
                    if (relu) acc[e] = acc[e] < 0.0f ? 0.0f : acc[e];  // keeps NaN, as torch.relu does
                }
                const int col = slab * kSlab + li * 4;
                float* __restrict__ zr = Zs + (int64_t)row * ldz;
                if (vec_out) {
                    if (col < d) store_vec<4>(zr, acc);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < d) zr[e] = acc[e];
                }
            }
        }
        // Short rows, a batch of kStep at a time: lane group `sub` owns row n_wide + b * kStep + sub of the
        // schedule and sums it alone, LPE entries per chunk -- its LPE lanes fetch one index each, every lane
        // then gathers all LPE rows of X (its own float4 of each) and adds them strictly in entry order.  The
        // groups of a wavefront walk in lockstep up to the longest row of the batch (the schedule sorts the
        // short rows by chunk count); entries past a row's end are clamped and get coefficient 0.  No sum
        // crosses lanes, and one round of loads serves kStep rows.
        for (int b = first; b * kStep < n - n_wide; b += stride) {
            const int di = n_wide + b * kStep + sub;
            const int4 dsc = di < n ? sched[di] : make_int4(0, 0, -1, 0);
            const int start = dsc.x, len = dsc.y - dsc.x;
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int c = 0; __builtin_amdgcn_ballot_w64(c < len) != 0; c += LPE) {
                const int kc = max(min(start + c + li, dsc.y - 1), 0);
                const uint32_t p_all = idx[kc];
                float f_all = 0.0f;
                if constexpr (COEF == kCoefStream) f_all = val[kc];
                uint32_t p[LPE];
                float f[LPE];
                float x[LPE][4];
#pragma unroll
                for (int e = 0; e < LPE; e++) {
                    p[e] = __shfl(p_all, lane - li + e, kWave);
                    if constexpr (COEF == kCoefStream) f[e] = __shfl(f_all, lane - li + e, kWave);
                }
#pragma unroll
                for (int e = 0; e < LPE; e++) {
                    const uint32_t col = p[e] & 0x7fffffffu;
                    if constexpr (COEF != kCoefStream) {
                        const uint32_t mag = COEF == kCoefSignM ? __float_as_uint(m[col]) : 0x3f800000u;
                        f[e] = __uint_as_float(mag ^ (p[e] & 0x80000000u));
                    }
                    f[e] = c + e < len ? f[e] : 0.0f;
                    load_vec<4>(Xs + (int64_t)col * x_row_stride, x[e]);
                }
#pragma unroll
                for (int e = 0; e < LPE; e++)
#pragma unroll
                    for (int q = 0; q < 4; q++) acc[q] = fmaf(f[e], x[e][q], acc[q]);
            }
            if (dsc.z >= 0) {
                const float row_scale = __int_as_float(dsc.w);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    acc[q] *= row_scale;
                    if (relu) acc[q] = acc[q] < 0.0f ? 0.0f : acc[q];
                }
                const int col = slab * kSlab + li * 4;
                float* __restrict__ zr = Zs + (int64_t)dsc.z * ldz;
                if (vec_out) {
                    if (col < d) store_vec<4>(zr, acc);
                } else {
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        if (col + q < d) zr[q] = acc[q];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// (1c) SpMM over blocks of entries that cluster: the rows are cut into panels of kPanelRows, the
// columns into tiles of TILE rows of X, and the entries of every (panel, tile) block that holds
// enough of them are stored apart ("local" entries) as 16-bit offsets into the tile.  A workgroup
// takes a (panel, slab) pair: for each of the panel's blocks it stages the tile's 128-byte slab of
// X rows in LDS and its 16 waves gather from there at LDS bandwidth, where the slab kernel pulls
// every 128-byte line through L1 and L2.
//   * Every 8-lane group of a wave owns ONE ROW of the panel (a wave works on 8 rows in lockstep,
//     2 such sets per wave = 256 rows per workgroup) and keeps that row's running sum in 4
//     registers per lane across all blocks: no cross-lane traffic at all, and a row's local
//     entries are added strictly in storage order (blocks by ascending tile, columns ascending).
//   * A lane group reads its row's entries as one 16-byte vector per 8 entries; every (row, block)
//     segment is padded to a multiple of 8 entries with the index of an all-zero row kept behind
//     the tile in LDS, and a group whose segment is shorter than its neighbours' gathers that row:
//     no coefficient, no masking -- per gather 1 address op (a 16-bit multiply-add on one half of
//     the index word), 1 ds_read_b128, 4 adds.
//   * lidx[k] = (row of X - first row of the tile) * 8 | sign << 15  (pre-multiplied so that the
//     byte offset into LDS is (lidx + float4 index of the lane) << 4).
// At the end the sums are added to what the slab kernel wrote for the remaining ("remote") entries
// of the row, scaled (left scale of the normalised multiply), passed through the ReLU if asked,
// and stored.  Order of the fp32 sums per output element: (remote part as the slab kernel sums
// it) + (local entries in storage order, starting from 0).
// ---------------------------------------------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));      // a native 16-byte vector (stays in registers)
constexpr int kPanelRows = CBM_TILING_PANEL_ROWS;           // rows of the matrix per panel
constexpr int kTiledWaves = 16;            // one 1024-thread workgroup

// LPE lanes serve one row: 8 for the 128-byte slabs, 4 for the 64-byte half slab of the last
// d % 32 columns (then 16 rows per wave in lockstep, one set per wave, and W / Z / d are those of
// the half slab: W its copy, Z already offset to its first column, d its width, n_slabs = 1).
// FUSED: the same lane group also gathers its row's REMOTE entries (rowptr_r / idx_r, packed like
// idx) straight from the slab-major copy in global memory once the panel's blocks are done, eight
// entries per row and set in flight, added strictly in order; nothing is read from Z and no launch
// of the slab kernel is needed.  While one workgroup waits on the fabric in that phase, the
// workgroups of other CUs are in their LDS phase: the two resources overlap across the chip.
// LDS byte address of a tile row for one lane: half `hi` of `word` holds (row of the tile) x 8; the row
// is LPE x 16 bytes long and `lane_lds` is the LDS address of the lane's float4 in row 0.
typedef const __attribute__((address_space(3))) f32x4* lds_f32x4_ptr;
template <int LPE>
__device__ __forceinline__ uint32_t lds_row_address(uint32_t word, int hi, uint32_t lane_lds) {
    static_assert(LPE == 8 || LPE == 4, "rows of 128 or 64 bytes");
    uint32_t at;
    if (LPE == 8) {
        if (hi) asm("v_mad_u32_u16 %0, %1, 16, %2 op_sel:[1,0,0,0]" : "=v"(at) : "v"(word), "v"(lane_lds));
        else asm("v_mad_u32_u16 %0, %1, 16, %2 op_sel:[0,0,0,0]" : "=v"(at) : "v"(word), "v"(lane_lds));
    } else {
        if (hi) asm("v_mad_u32_u16 %0, %1, 8, %2 op_sel:[1,0,0,0]" : "=v"(at) : "v"(word), "v"(lane_lds));
        else asm("v_mad_u32_u16 %0, %1, 8, %2 op_sel:[0,0,0,0]" : "=v"(at) : "v"(word), "v"(lane_lds));
    }
    return at;
}

template <int TILE, bool SIGNED, int LPE, bool FUSED>
__global__ __launch_bounds__(kWave * kTiledWaves) __attribute__((amdgpu_waves_per_eu(4, 4))) void spmm_tiled_local(
    const int32_t* __restrict__ panel_ptr, const int32_t* __restrict__ blk_tile, const int32_t* __restrict__ seg,
    const uint16_t* __restrict__ lidx, const int32_t* __restrict__ rowptr_r, const uint32_t* __restrict__ idx_r,
    const float* __restrict__ W, float* __restrict__ Z,
    const float* __restrict__ row_scale, int n, int d, int n_slabs, int n_panels, int64_t ldz, int relu, int vec_out) {
    constexpr int kGroups = kWave / LPE;                   // rows a wave serves in lockstep
    constexpr int kTiledSets = kPanelRows / (kTiledWaves * kGroups);
    constexpr int kRowFloats = LPE * 4;
    extern __shared__ float4 tile_lds[];                   // (TILE + 1) x LPE float4; row TILE is all zero
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = lane / LPE, li = lane % LPE;
    if (threadIdx.x < LPE) tile_lds[TILE * LPE + threadIdx.x] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    constexpr uint32_t kPad = (uint32_t)(TILE * 8) | ((uint32_t)(TILE * 8) << 16);    // two entries of the zero row
    const uint32_t lane_lds = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) float4*)tile_lds + li);
    // Workgroup b runs on XCD b % 8.  Items (panel-major, slab-minor) are cut into 8 contiguous
    // ranges, one per XCD, and dealt cyclically to the XCD's workgroups: the workgroups of an XCD
    // work on neighbouring panels at the same time, which share their tiles through the XCD's L2.
    const int xcd = blockIdx.x % kXcds, j0 = blockIdx.x / kXcds, G = gridDim.x / kXcds;
    const int items = n_panels * n_slabs;
    const int chunk = (items + kXcds - 1) / kXcds;
    const int item_end = min((xcd + 1) * chunk, items);
    for (int item = xcd * chunk + j0; item < item_end; item += G) {
        const int panel = item / n_slabs, slab = item % n_slabs;
        float acc[kTiledSets][4];
#pragma unroll
        for (int t = 0; t < kTiledSets; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[t][e] = 0.0f;
        const int b_beg = panel_ptr[panel], b_end = panel_ptr[panel + 1];
        // The tile of block b + 1 is fetched into registers while block b is gathered from LDS, so
        // that between two blocks only the LDS stores and two barriers are exposed.
        constexpr int kStage = TILE * LPE / (kWave * kTiledWaves);        // float4 per thread and tile
        f32x4 stage[kStage];
#define CBM_FETCH_TILE(B)                                                                                            \
    do {                                                                                                             \
        const int base_ = blk_tile[B] * TILE;                                                                        \
        const int rows8_ = min(TILE, n - base_) * LPE;                                                               \
        const f32x4* __restrict__ src_ = reinterpret_cast<const f32x4*>(W + ((int64_t)slab * n + base_) * kRowFloats); \
        _Pragma("unroll") for (int i_ = 0; i_ < kStage; i_++)   /* all loads in flight together; rows past the */    \
            stage[i_] = src_[min(i_ * (kWave * kTiledWaves) + (int)threadIdx.x, rows8_ - 1)]; /* matrix: never gathered */ \
    } while (0)
        if (b_beg < b_end) CBM_FETCH_TILE(b_beg);
        for (int b = b_beg; b < b_end; b++) {
            // this lane group's segment in each set: panel row = set * (16 waves x rows per wave) + wave * rows per wave
            // + lane group; seg[] counts in units of 8 entries
            int s0[kTiledSets], len[kTiledSets];
#pragma unroll
            for (int t = 0; t < kTiledSets; t++) {
                const int32_t* __restrict__ sg = seg + (int64_t)b * (kPanelRows + 1) + t * (kTiledWaves * kGroups) + wave * kGroups + sub;
                s0[t] = sg[0]; len[t] = sg[1] - s0[t];
            }
            __syncthreads();                               // the previous tile is no longer read
#pragma unroll
            for (int i = 0; i < kStage; i++)
                reinterpret_cast<f32x4*>(tile_lds)[i * (kWave * kTiledWaves) + threadIdx.x] = stage[i];
            __syncthreads();
            if (b + 1 < b_end) CBM_FETCH_TILE(b + 1);
#pragma unroll
            for (int t = 0; t < kTiledSets; t++) {
                int longest = len[t];                       // the wave iterates to its longest segment
#pragma unroll
                for (int off = LPE; off < kWave; off <<= 1) longest = max(longest, __shfl_xor(longest, off, kWave));
                longest = __builtin_amdgcn_readfirstlane(longest);
                const uint4* __restrict__ mine = reinterpret_cast<const uint4*>(lidx) + s0[t];
                const uint4 pad4 = make_uint4(kPad, kPad, kPad, kPad);
                // 8 entries = one 16-byte vector; gathers, then adds in entry order
                auto gather8 = [&](const uint4& v) {
                    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                    f32x4 x[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        // byte address in LDS = (row of the tile x 8) x (2 LPE) + 16 x lane of the group: one
                        // 16-bit multiply-add on the selected half of the index word
                        const uint32_t word = SIGNED ? (w[u >> 1] & 0x7fff7fffu) : w[u >> 1];
                        x[u] = *reinterpret_cast<lds_f32x4_ptr>(lds_row_address<LPE>(word, u & 1, lane_lds));
                    }
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        if constexpr (SIGNED) {
                            const uint32_t p = (u & 1) ? (w[u >> 1] >> 16) : (w[u >> 1] & 0xffffu);
                            const float f = __uint_as_float(0x3f800000u | ((p & 0x8000u) << 16));
                            acc[t][0] = fmaf(f, x[u][0], acc[t][0]); acc[t][1] = fmaf(f, x[u][1], acc[t][1]);
                            acc[t][2] = fmaf(f, x[u][2], acc[t][2]); acc[t][3] = fmaf(f, x[u][3], acc[t][3]);
                        } else {
                            acc[t][0] += x[u][0]; acc[t][1] += x[u][1]; acc[t][2] += x[u][2]; acc[t][3] += x[u][3];
                        }
                    }
                };
                // four index vectors (32 entries) are requested together, then gathered: one wait per
                // 32 gathers; the other wavefronts of the SIMD cover it
                for (int j = 0; j < longest; j += CBM_TILED_VECS) {
                    uint4 v[CBM_TILED_VECS];
#pragma unroll
                    for (int q = 0; q < CBM_TILED_VECS; q++) {
                        v[q] = pad4;
                        if (j + q < len[t]) v[q] = mine[j + q];
                    }
#pragma unroll
                    for (int q = 0; q < CBM_TILED_VECS; q++)
                        if (j + q < longest) gather8(v[q]);
                }
            }
        }
#undef CBM_FETCH_TILE
        float racc[kTiledSets][4];                         // FUSED: the remote entries' sum, in entry order
        if constexpr (FUSED) {
            int rs[kTiledSets], rn[kTiledSets], longest = 0;
#pragma unroll
            for (int t = 0; t < kTiledSets; t++) {
                const int row = panel * kPanelRows + t * (kTiledWaves * kGroups) + wave * kGroups + sub;
                rs[t] = 0; rn[t] = 0;
                if (row < n) { rs[t] = rowptr_r[row]; rn[t] = rowptr_r[row + 1] - rs[t]; }
                longest = max(longest, rn[t]);
#pragma unroll
                for (int e = 0; e < 4; e++) racc[t][e] = 0.0f;
            }
#pragma unroll
            for (int off = LPE; off < kWave; off <<= 1) longest = max(longest, __shfl_xor(longest, off, kWave));
            longest = __builtin_amdgcn_readfirstlane(longest);
            // uniform base of the slab + 32-bit byte offset per lane (the host checks n * 16 LPE < 2^32)
            const char* __restrict__ Ws = reinterpret_cast<const char*>(W + (int64_t)slab * n * kRowFloats);
            const uint32_t lane_off = (uint32_t)li * 16u;
            // entries per row in flight: the registers of the LDS phase are free here
            constexpr int kRU = LPE == 8 ? CBM_TILED_REMOTE_U8 : CBM_TILED_REMOTE_U4;
            constexpr int kPer = (kRU + LPE - 1) / LPE;    // index words per lane and round
            // word q of lane li of a group holds entry k + q * LPE + li of the group's row; next
            // round's indices are requested before this round's rows
            uint32_t mine[kTiledSets][kPer], nxt[kTiledSets][kPer];
            auto fetch_idx = [&](int k, uint32_t (&out)[kTiledSets][kPer]) {
#pragma unroll
                for (int t = 0; t < kTiledSets; t++)
#pragma unroll
                    for (int q = 0; q < kPer; q++) {
                        const int kk = k + q * LPE + li;
                        out[t][q] = (q * LPE + li < kRU && kk < rn[t]) ? idx_r[rs[t] + kk] : 0u;
                    }
            };
            if (longest > 0) fetch_idx(0, nxt);
            for (int k = 0; k < longest; k += kRU) {
#pragma unroll
                for (int t = 0; t < kTiledSets; t++)
#pragma unroll
                    for (int q = 0; q < kPer; q++) mine[t][q] = nxt[t][q];
                if (k + kRU < longest) fetch_idx(k + kRU, nxt);
                f32x4 x[kTiledSets][kRU];
                uint32_t p[kTiledSets][kRU];
#pragma unroll
                for (int t = 0; t < kTiledSets; t++)
#pragma unroll
                    for (int u = 0; u < kRU; u++) {
                        p[t][u] = (uint32_t)__shfl((int)mine[t][u / LPE], (lane & ~(LPE - 1)) + (u % LPE), kWave);
                        // past the row's end: row 0, masked below
                        x[t][u] = *reinterpret_cast<const f32x4*>(Ws + ((p[t][u] & 0x7fffffffu) * (uint32_t)(LPE * 16) + lane_off));
                    }
#pragma unroll
                for (int t = 0; t < kTiledSets; t++)
#pragma unroll
                    for (int u = 0; u < kRU; u++) {
                        const bool live = k + u < rn[t];
                        const float f = SIGNED ? __uint_as_float(0x3f800000u | (p[t][u] & 0x80000000u)) : 1.0f;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float v = live ? x[t][u][e] : 0.0f;
                            racc[t][e] = SIGNED ? fmaf(f, v, racc[t][e]) : racc[t][e] + v;
                        }
                    }
            }
        }
        // epilogue: every lane group adds its row's local sum to the remote part
#pragma unroll
        for (int t = 0; t < kTiledSets; t++) {
            const int row = panel * kPanelRows + t * (kTiledWaves * kGroups) + wave * kGroups + sub;
            const int col = slab * kRowFloats + li * 4;
            if (row < n && col < d) {
                float* __restrict__ zr = Z + (int64_t)row * ldz + col;
                const float sc = row_scale ? row_scale[row] : 1.0f;
                if constexpr (FUSED) {
                    float z[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        z[e] = (racc[t][e] + acc[t][e]) * sc;
                        if (relu) z[e] = z[e] < 0.0f ? 0.0f : z[e];
                    }
                    if (vec_out) {
                        *reinterpret_cast<float4*>(zr) = make_float4(z[0], z[1], z[2], z[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (col + e < d) zr[e] = z[e];
                    }
                } else if (vec_out) {
                    float4 z = *reinterpret_cast<const float4*>(zr);
                    z.x = (z.x + acc[t][0]) * sc; z.y = (z.y + acc[t][1]) * sc;
                    z.z = (z.z + acc[t][2]) * sc; z.w = (z.w + acc[t][3]) * sc;
                    if (relu) {
                        z.x = z.x < 0.0f ? 0.0f : z.x; z.y = z.y < 0.0f ? 0.0f : z.y;
                        z.z = z.z < 0.0f ? 0.0f : z.z; z.w = z.w < 0.0f ? 0.0f : z.w;
                    }
                    *reinterpret_cast<float4*>(zr) = z;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < d) {
                            float z = (zr[e] + acc[t][e]) * sc;
                            if (relu) z = z < 0.0f ? 0.0f : z;
                            zr[e] = z;
                        }
                }
            }
        }
    }
}

// Slab-major copy of X: W[s][r][0 .. 32) = X[r][32 s .. 32 s + 32), zero where the column is >= d
// (n_slabs * 32 may exceed d).  With the caller's row-major X a slab's lines sit a whole row (a
// power of two for the usual widths) apart, which maps them onto a fraction of an XCD's L2
// channels, and rows of odd widths are not line-aligned at all; in the copy the lines of a slab
// are consecutive and aligned.  One thread per float4 of the copy.
// With a mask matrix M (same shape as X, row stride ldm) the copy holds X where M > 0 and zero
// elsewhere: the gradient of a ReLU applied to the incoming gradient in the pass that copies it.
// With a scale vector the copy holds scale[r] * X[r][:] (one correctly rounded fp32 product per
// element): the right-hand diagonal of D^-1/2 (A + I) D^-1/2 applied once per row of X instead of
// once per delta entry, after which the SpMM needs no coefficient per entry, only the sign bit.
template <bool VEC_IN, bool MASKED, bool SCALED>
__global__ __launch_bounds__(256) void relayout_slabs(const float* __restrict__ X, float* __restrict__ W, int n, int d,
                                                      int n_slabs, int tail4, int64_t ldx, const float* __restrict__ M,
                                                      int64_t ldm, const float* __restrict__ scale) {
    // n_slabs full slabs of 8 float4 per row, then (tail4 = 4) one half slab of 4 float4 per row,
    // stored behind all full slabs: W[s][r][0 .. 32) for s < n_slabs, then T[r][0 .. 16).
    constexpr int kSlab4 = 8;                              // float4 per 128-byte slab
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int row4 = n_slabs * kSlab4 + tail4;
    if (t >= (int64_t)n * row4) return;
    const int r = (int)(t / row4), q = (int)(t % row4);
    const int s = q / kSlab4, w = q % kSlab4;
    const int col = 4 * q;
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    const float* __restrict__ src = X + (int64_t)r * ldx + col;
    if constexpr (VEC_IN) {
        if (col < d) v = *reinterpret_cast<const float4*>(src);
    } else {
        if (col + 0 < d) v.x = src[0];
        if (col + 1 < d) v.y = src[1];
        if (col + 2 < d) v.z = src[2];
        if (col + 3 < d) v.w = src[3];
    }
    if constexpr (MASKED) {
        const float* __restrict__ msk = M + (int64_t)r * ldm + col;
        float4 k = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if constexpr (VEC_IN) {
            if (col < d) k = *reinterpret_cast<const float4*>(msk);
        } else {
            if (col + 0 < d) k.x = msk[0];
            if (col + 1 < d) k.y = msk[1];
            if (col + 2 < d) k.z = msk[2];
            if (col + 3 < d) k.w = msk[3];
        }
        v.x = k.x > 0.0f ? v.x : 0.0f; v.y = k.y > 0.0f ? v.y : 0.0f;
        v.z = k.z > 0.0f ? v.z : 0.0f; v.w = k.w > 0.0f ? v.w : 0.0f;
    }
    if constexpr (SCALED) {
        const float f = scale[r];
        v.x *= f; v.y *= f; v.z *= f; v.w *= f;
    }
    float* __restrict__ dst = s < n_slabs ? W + (((int64_t)s * n + r) * kSlab4 + w) * 4
                                          : W + (int64_t)n * n_slabs * 32 + ((int64_t)r * tail4 + w) * 4;
    *reinterpret_cast<float4*>(dst) = v;
}

// coef[k] = +-m[col(k)]: the packed entries expanded once so the SpMM can stream coefficients.
__global__ __launch_bounds__(256) void expand_coef(const uint32_t* __restrict__ idx, const float* __restrict__ m,
                                                   float* __restrict__ coef, int64_t nnz) {
    const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= nnz) return;
    const uint32_t p = idx[k];
    coef[k] = __uint_as_float(__float_as_uint(m[p & 0x7fffffffu]) ^ (p & 0x80000000u));
}

// ---------------------------------------------------------------------------------------------
// (2) propagate: one row v = order[i], parent u.  dv = d - d % 8 separates the reference's
// FMA vector body from its scalar tail (cbm_extensions.cpp:966-990).
// ---------------------------------------------------------------------------------------------
template <int VEC, int CH, bool NORM, bool FULL>
__device__ __forceinline__ void propagate_row(int v, int u, const float* __restrict__ m, float* __restrict__ Y,
                                              int d, int dv, int64_t ldy, int col0) {
    float mu = 1.0f, mv = 1.0f, inv_mu = 1.0f;
    if constexpr (NORM) { mu = m[u]; mv = m[v]; inv_mu = 1.0f / mu; }
    const float* __restrict__ yu = Y + (int64_t)u * ldy + col0;
    float* __restrict__ yv = Y + (int64_t)v * ldy + col0;
    float a[CH][VEC], b[CH][VEC];
#pragma unroll
    for (int c = 0; c < CH; c++)
        if (FULL || col0 + c * kWave * VEC < d) {
            load_vec<VEC>(yu + c * kWave * VEC, a[c]);
            load_vec<VEC>(yv + c * kWave * VEC, b[c]);
        }
#pragma unroll
    for (int c = 0; c < CH; c++)
        if (FULL || col0 + c * kWave * VEC < d) {
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if constexpr (NORM) {
                    const int j = col0 + c * kWave * VEC + e;
                    b[c][e] = (j < dv) ? fmaf(a[c][e], inv_mu, b[c][e]) * mv : (b[c][e] + a[c][e] / mu) * mv;
                } else {
                    b[c][e] += a[c][e];
                }
            }
            store_vec<VEC>(yv + c * kWave * VEC, b[c]);
        }
}

template <int VEC, int CH, bool NORM, bool FULL>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void propagate_level(
    const int32_t* __restrict__ parent, const int32_t* __restrict__ order, int beg, int end,
    const float* __restrict__ m, float* __restrict__ Y, int d, int dv, int64_t ldy) {
    const int lane = threadIdx.x & (kWave - 1);
    const int i = beg + blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (i >= end) return;
    const int v = __builtin_amdgcn_readfirstlane(order[i]);
    const int u = __builtin_amdgcn_readfirstlane(parent[v]);
    propagate_row<VEC, CH, NORM, FULL>(v, u, m, Y, d, dv, ldy, blockIdx.y * (kWave * VEC * CH) + lane * VEC);
}

// A run of narrow levels [l_beg, l_end) handled by ONE workgroup: its 16 waves share each level's
// rows (at most kNarrowWidth = 64, so at most 4 per wave) and meet at a barrier between levels.
// The (row, parent) pairs of the NEXT level do not depend on Y, so each wave fetches them before
// the barrier; after it only the two Y rows are on the critical path.  All waves of a workgroup
// share one L1, so a workgroup-scope fence orders the stores of one level before the loads of
// the next.  Column tiles (grid.y) are independent: every tile is its own single workgroup.
template <int VEC, int CH, bool NORM, bool FULL>
__global__ __launch_bounds__(kWave * kNarrowWaves) void propagate_narrow_levels(
    const int32_t* __restrict__ parent, const int32_t* __restrict__ order,
    const int32_t* __restrict__ level_off, int l_beg, int l_end, const float* __restrict__ m,
    float* __restrict__ Y, int d, int dv, int64_t ldy) {
    constexpr int kPerWave = kNarrowWidth / kNarrowWaves;        // rows of a level one wave may own
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int col0 = blockIdx.y * (kWave * VEC * CH) + lane * VEC;
    // lane t < kPerWave of a wave holds the wave's t-th row of the level (and its parent)
    auto fetch = [&](int l, int& v, int& u) {
        v = -1; u = -1;
        if (l < l_end && lane < kPerWave) {
            const int i = level_off[l] + wave + kNarrowWaves * lane;
            if (i < level_off[l + 1]) { v = order[i]; u = parent[v]; }
        }
    };
    int my_v, my_u;
    fetch(l_beg, my_v, my_u);
    for (int l = l_beg; l < l_end; l++) {
        const int cur_v = my_v, cur_u = my_u;
        fetch(l + 1, my_v, my_u);
#pragma unroll
        for (int t = 0; t < kPerWave; t++) {
            const int v = bcast_i(cur_v, t);
            if (v < 0) break;
            propagate_row<VEC, CH, NORM, FULL>(v, bcast_i(cur_u, t), m, Y, d, dv, ldy, col0);
        }
        __threadfence_block();
        __syncthreads();
    }
}

// A run of levels that all hold ONE row is a chain: row k's parent is row k - 1 of the run.  One
// thread per feature column carries the running value in a register down the chain, so the only
// dependency between levels is an add; the rows of Y it needs are independent loads.  The chain is
// walked in stretches of 64 levels -- the 64 row ids (and their m) of a stretch come in with one
// coalesced load and are broadcast with v_readlane -- and every stretch in two halves: while one
// half's 32 rows are added, the loads of the next half are in flight, and the ids of the stretch
// after the next are already requested, so that no load is waited for right after it is issued.
// All loads are unconditional (past the end of the chain: the chain's first row again) -- a load
// that may or may not have been issued would force the wait in front of the next add down to
// zero.  Arithmetic per level is exactly that of propagate_row.
constexpr int kChainHalf = 32;
constexpr int kMinChain = 4;               // shorter runs of single-row levels stay with the other kernels

template <bool NORM>
__global__ __launch_bounds__(kWave * kNarrowWaves) void propagate_chain(
    const int32_t* __restrict__ parent, const int32_t* __restrict__ order, int first, int count,
    const float* __restrict__ m, float* __restrict__ Y, int d, int dv, int64_t ldy) {
    static_assert(2 * kChainHalf == kWave, "a stretch is one row id per lane");
    const int lane = threadIdx.x & (kWave - 1);
    const int j = blockIdx.x * blockDim.x + threadIdx.x;          // feature column of this thread
    const bool live = j < d;                                      // whole waves beyond d were not launched
    const int jj = live ? j : 0;                                  // lanes past d (last wavefront only) load column 0 and store nothing
    const int v0 = order[first];
    const int u0 = parent[v0];
    float run = Y[(int64_t)u0 * ldy + jj];                         // final value of the row above the chain
    float mu = NORM ? m[u0] : 1.0f;
    // ids of the stretch that starts at level `base`, one per lane; v0 past the end of the chain
    auto ids = [&](int base) -> int {
        const int g = min(base + lane, count - 1);
        const int v = order[first + g];
        return base + lane < count ? v : v0;
    };
    // A level's row of Y starts at Y + v * ldy: the lane that holds v computes the offset once per stretch, and a
    // level gets it with two v_readlane into a scalar pair (the address of a load is then scalar base + lane column)
    // instead of a 64-bit scalar multiply per load and per store.
    auto row_of = [&](int64_t off_ids, int k) -> char* {         // off_ids: byte offsets v * ldy * 4, one per lane
        const uint32_t lo = (uint32_t)bcast_i((int)(uint32_t)off_ids, k);
        const uint32_t hi = (uint32_t)bcast_i((int)(uint32_t)((uint64_t)off_ids >> 32), k);
        return reinterpret_cast<char*>(Y) + (int64_t)(((uint64_t)hi << 32) | lo);
    };
    const uint32_t jj4 = (uint32_t)jj * 4u;                      // scalar row address + unsigned 32-bit byte offset of the lane
    auto request = [&](float (&z)[kChainHalf], int64_t off_ids, int half) {
#pragma unroll
        for (int u = 0; u < kChainHalf; u++) z[u] = *reinterpret_cast<const float*>(row_of(off_ids, half * kChainHalf + u) + jj4);
    };
    // `full`: every level of this half exists (no test per level; the last stretches of a chain take the other path)
    auto consume = [&](auto full, const float (&z)[kChainHalf], int64_t off_ids, float m_ids, int base, int half) {
#pragma unroll
        for (int u = 0; u < kChainHalf; u++) {
            const int k = half * kChainHalf + u;
            if (decltype(full)::value || base + k < count) {
                if constexpr (NORM) {
                    const float mv = bcast_f(m_ids, k);
                    const float inv_mu = 1.0f / mu;
                    run = (jj < dv) ? fmaf(run, inv_mu, z[u]) * mv : (z[u] + run / mu) * mv;
                    mu = mv;
                } else {
                    run = z[u] + run;
                }
                // lanes past d carry column 0 along but must not store it: the wavefront that owns column 0 may
                // not have loaded this row yet
                if (live) *reinterpret_cast<float*>(row_of(off_ids, k) + jj4) = run;
            }
        }
    };
    int v_cur = ids(0), v_nxt = ids(kWave);
    int64_t o_cur = (int64_t)v_cur * ldy * 4, o_nxt = (int64_t)v_nxt * ldy * 4;
    float m_cur = 1.0f;
    if constexpr (NORM) m_cur = m[v_cur];
    float za[kChainHalf], zb[kChainHalf];
    request(za, o_cur, 0);
    for (int base = 0; base < count; base += kWave) {
        // requested first, needed last (by then older than every load still in flight): the ids of the stretch
        // after the next, and the m of the next stretch's rows (their ids came in an iteration ago)
        const int v_far = ids(base + 2 * kWave);
        float m_nxt = 1.0f;
        if constexpr (NORM) m_nxt = m[v_nxt];
        request(zb, o_cur, 1);
        if (base + kWave <= count) {
            consume(std::true_type{}, za, o_cur, m_cur, base, 0);
            request(za, o_nxt, 0);
            consume(std::true_type{}, zb, o_cur, m_cur, base, 1);
        } else {
            consume(std::false_type{}, za, o_cur, m_cur, base, 0);
            request(za, o_nxt, 0);
            consume(std::false_type{}, zb, o_cur, m_cur, base, 1);
        }
        v_nxt = v_far;
        o_cur = o_nxt; m_cur = m_nxt;
        o_nxt = (int64_t)v_far * ldy * 4;
    }
}

// The walk of all subtrees below a level in ONE launch (plan: cbm_walk_plan_build).  A wavefront takes a bin
// of the plan -- whole subtrees, each a sequence of rows in depth-first pre-order -- and 64 feature columns
// (one per lane), and carries the value of the row it has just finished in a register: the next row of the
// sequence is usually that row's first child.  A row with two or more children also leaves its value (with
// its m and 1 / m) in an LDS slot of the wavefront, where the later children find it; children are ordered lightest
// subtree first, so few slots are live at once.  Global memory is touched twice per row -- its SpMM result is
// read, its final value written -- and no load depends on an earlier store, so, as in propagate_chain, the
// rows of a stretch of 64 entries are requested half a stretch ahead and every load is unconditional (past
// the end of the bin: the bin's first row again).  The head of a subtree is final already (a child of the
// root after the SpMM, or a row of a level walked before this launch): it is loaded, not stored.
// Arithmetic per row is exactly that of propagate_row, so Y is bit-identical to the level-by-level walk.
constexpr int kSubWaves = 4;               // wavefronts per workgroup (each owns its LDS slots)
constexpr int kSlotFloats = 3 * kWave;     // a slot: a row's value, its m and 1 / m, per feature column of the wavefront

template <bool NORM>
__global__ __launch_bounds__(kWave * kSubWaves) void propagate_subtrees(
    const int2* __restrict__ entries, const int32_t* __restrict__ bin_off, int n_bins, int slices,
    const float* __restrict__ m, float* __restrict__ Y, int d, int dv, int64_t ldy, int n_slots) {
    extern __shared__ float walk_slots[];                         // [kSubWaves][n_slots][3][64]
    const int lane = threadIdx.x & (kWave - 1);
    const int w = blockIdx.x * kSubWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform, and
    const int bin = w / slices;                                                                // known to be
    if (bin >= n_bins) return;
    const int j0 = (w % slices) * kWave;                          // first feature column of this wavefront
    const int j = j0 + lane;                                      // feature column of this thread
    const bool live = j < d;
    const int jj = live ? j : 0;                                  // lanes past d load column 0 and store nothing
    const bool all_body = j0 + kWave <= dv;     // wave-uniform: no column of the division tail in this wavefront
    const bool all_live = j0 + kWave <= d;      // wave-uniform: every lane stores
    float* __restrict__ st = walk_slots + (size_t)(threadIdx.x >> 6) * n_slots * kSlotFloats + lane;
    const int first = __builtin_amdgcn_readfirstlane(bin_off[bin]);
    const int count = __builtin_amdgcn_readfirstlane(bin_off[bin + 1]) - first;
    const int2 e0 = entries[first];
    auto ids = [&](int base) -> int2 {                            // entry base + lane; past the end: the first one
        const int2 e = entries[first + min(base + lane, count - 1)];
        return base + lane < count ? e : e0;
    };
    typedef __attribute__((address_space(1))) char* global_bytes;      // device memory, not a flat address
    typedef __attribute__((address_space(1))) float* global_float;
    // what lane l keeps for entry l of a stretch: the address of its row of Y (wave-uniform once broadcast: a
    // load or store then has a scalar base and the lane's column offset)
    auto row_addr = [&](int row) -> uint64_t {
        return (uint64_t)reinterpret_cast<uintptr_t>(Y) + (uint64_t)(uint32_t)row * (uint64_t)ldy * 4u;
    };
    const uint32_t jj4 = (uint32_t)jj * 4u;
    auto row_of = [&](uint64_t addr_ids, int k) -> global_float {
        const uint32_t lo = (uint32_t)bcast_i((int)(uint32_t)addr_ids, k);
        const uint32_t hi = (uint32_t)bcast_i((int)(uint32_t)(addr_ids >> 32), k);
        return (global_float)((global_bytes)(uintptr_t)(((uint64_t)hi << 32) | lo) + jj4);
    };
    auto request = [&](float (&z)[kChainHalf], uint64_t addr_ids, int half) {
#pragma unroll
        for (int u = 0; u < kChainHalf; u++) z[u] = *row_of(addr_ids, half * kChainHalf + u);
    };
    // mu, inv_mu: m of the row just finished and 1 / it (the reference divides once per row, cpp:1329-1354:
    // here lane l does that division for the l-th row of a stretch, all 64 at once)
    float run = 0.0f, mu = 1.0f, inv_mu = 1.0f;
    auto consume = [&](auto full, const float (&z)[kChainHalf], uint64_t addr_ids, int c_ids, float m_ids, float im_ids, int base,
                       int half) {
        // A half stretch of plain chain steps (every control word 0: the parent is the row before, nothing to
        // keep) in a wavefront without tail columns or idle lanes: no test per row.  Past the end of the bin the
        // control words are those of the bin's head (never 0), so a partial stretch never comes here.
        const uint64_t not_plain = __builtin_amdgcn_ballot_w64(c_ids != 0);
        if (((not_plain >> (half * kChainHalf)) & 0xffffffffull) == 0 && all_live && (!NORM || all_body)) {
#pragma unroll
            for (int u = 0; u < kChainHalf; u++) {
                const int k = half * kChainHalf + u;
                if constexpr (NORM) {
                    const float mv = bcast_f(m_ids, k);
                    run = fmaf(run, inv_mu, z[u]) * mv;
                    mu = mv;
                    inv_mu = bcast_f(im_ids, k);
                } else {
                    run = z[u] + run;
                }
                *row_of(addr_ids, k) = run;
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < kChainHalf; u++) {
            const int k = half * kChainHalf + u;
            if (decltype(full)::value || base + k < count) {
                const int ctl = bcast_i(c_ids, k);                // wave-uniform: the branches below are scalar
                const int src = ctl & 63, dst = (ctl >> 8) & 63;
                const float mv = NORM ? bcast_f(m_ids, k) : 1.0f;
                if (src == CBM_WALK_LOAD_ONLY) {
                    run = z[u];
                } else {
                    float a = run, ma = mu, inv = inv_mu;
                    if (src) {
                        a = st[(src - 1) * kSlotFloats];
                        if constexpr (NORM) { ma = st[(src - 1) * kSlotFloats + kWave]; inv = st[(src - 1) * kSlotFloats + 2 * kWave]; }
                    }
                    if constexpr (NORM) {
                        if (all_body) run = fmaf(a, inv, z[u]) * mv;
                        else run = (jj < dv) ? fmaf(a, inv, z[u]) * mv : (z[u] + a / ma) * mv;
                    } else {
                        run = z[u] + a;
                    }
                    if (live) *row_of(addr_ids, k) = run;
                }
                mu = mv;
                if constexpr (NORM) inv_mu = bcast_f(im_ids, k);
                if (dst) {
                    st[(dst - 1) * kSlotFloats] = run;
                    if constexpr (NORM) { st[(dst - 1) * kSlotFloats + kWave] = mv; st[(dst - 1) * kSlotFloats + 2 * kWave] = bcast_f(im_ids, k); }
                }
            }
        }
    };
    int2 e_cur = ids(0), e_nxt = ids(kWave);
    uint64_t a_cur = row_addr(e_cur.x), a_nxt = row_addr(e_nxt.x);
    float m_cur = 1.0f, im_cur = 1.0f;
    if constexpr (NORM) { m_cur = m[e_cur.x]; im_cur = 1.0f / m_cur; }
    float za[kChainHalf], zb[kChainHalf];
    request(za, a_cur, 0);
    for (int base = 0; base < count; base += kWave) {
        const int2 e_far = ids(base + 2 * kWave);
        float m_nxt = 1.0f;
        if constexpr (NORM) m_nxt = m[e_nxt.x];
        request(zb, a_cur, 1);
        if (base + kWave <= count) {
            consume(std::true_type{}, za, a_cur, e_cur.y, m_cur, im_cur, base, 0);
            request(za, a_nxt, 0);
            consume(std::true_type{}, zb, a_cur, e_cur.y, m_cur, im_cur, base, 1);
        } else {
            consume(std::false_type{}, za, a_cur, e_cur.y, m_cur, im_cur, base, 0);
            request(za, a_nxt, 0);
            consume(std::false_type{}, zb, a_cur, e_cur.y, m_cur, im_cur, base, 1);
        }
        e_cur = e_nxt; e_nxt = e_far;
        a_cur = a_nxt; m_cur = m_nxt;
        if constexpr (NORM) im_cur = 1.0f / m_cur;
        a_nxt = row_addr(e_far.x);
    }
}

// The whole multiply of a DEEP tree with SHORT delta rows in one launch: the walk of propagate_subtrees with
// the SpMM result of a row summed on the spot instead of read back.  The host lays the delta entries of a
// bin's rows end to end in the order the walk visits them (gidx: col | sign << 31, CBM_STREAM_LAST on a row's
// last entry, CBM_STREAM_DUMMY on the one stand-in entry of an empty row) and pads the bin to whole stretches
// of 64 entries; a wavefront streams that list a stretch at a time, lane l decoding entry l (its coefficient
// +-1 or +-m[col], the address of row col of X), and gathers its 64 feature columns of every entry's row a
// whole stretch ahead of their use: entry k's register is re-used for entry k of the next stretch as soon as
// it has been added, so 64 gathers are in flight all the time and no load is conditional.  The sum of a row
// runs strictly in entry order (fma(coef, x, acc) from zero: the order of spmm_wave_per_row); when its last
// entry is in, the row takes its walk step exactly as in propagate_subtrees (the head of a subtree is a child
// of the root: its sum times m) and is stored once -- through the ReLU if asked, the raw value staying in the
// register / LDS slot its children read.  ginfo holds, per stretch, the {row, ctl} of the rows that end inside
// it, in order.  Everything that steers control flow is wave-uniform (scalar branches, the common case falls
// through).  Z never exists in memory.
constexpr uint32_t kStreamLast = CBM_STREAM_LAST, kStreamDummy = CBM_STREAM_DUMMY, kStreamCol = CBM_STREAM_COL_MASK;

template <bool NORM>
__global__ __launch_bounds__(kWave * kSubWaves) void spmm_update_subtrees(
    const uint32_t* __restrict__ gidx, const int2* __restrict__ ginfo, const int32_t* __restrict__ bin_goff, int n_bins,
    int slices, const float* __restrict__ m, const float* __restrict__ X, float* __restrict__ Y, int d, int dv, int64_t ldx,
    int64_t ldy, int n_slots, int relu) {
    extern __shared__ float walk_slots[];                         // [kSubWaves][n_slots][3][64]
    const int lane = threadIdx.x & (kWave - 1);
    const int w = blockIdx.x * kSubWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform, and
    const int bin = w / slices;                                                                // known to be
    if (bin >= n_bins) return;
    const int j0 = (w % slices) * kWave;                          // first feature column of this wavefront
    const int j = j0 + lane;                                      // feature column of this thread
    const bool live = j < d;
    const int jj = live ? j : 0;                                  // lanes past d gather column 0 and store nothing
    const bool all_body = j0 + kWave <= dv;     // wave-uniform: no column of the division tail in this wavefront
    float* __restrict__ st = walk_slots + (size_t)(threadIdx.x >> 6) * n_slots * kSlotFloats + lane;
    const int first = __builtin_amdgcn_readfirstlane(bin_goff[bin]);
    const int count = __builtin_amdgcn_readfirstlane(bin_goff[bin + 1]) - first;       // a multiple of 64
    auto at = [&](int base) -> int { return first + min(base, count - kWave) + lane; };   // past the end: the last stretch
    const uint32_t jj4 = (uint32_t)jj * 4u;
    // what lane l keeps for entry l of a stretch: the address of its row of X (wave-uniform once broadcast:
    // the gather then is one load with a scalar base and the lane's column offset)
    auto x_row = [&](uint32_t p) -> uint64_t {
        return (uint64_t)reinterpret_cast<uintptr_t>(X) + (uint64_t)(p & kStreamCol) * (uint64_t)ldx * 4u;
    };
    auto coef = [&](uint32_t p) -> float {
        uint32_t mag = 0x3f800000u;
        if constexpr (NORM) mag = __float_as_uint(m[p & kStreamCol]);
        return __uint_as_float(mag ^ (p & 0x80000000u));
    };
    auto gather = [&](uint64_t xr_ids, int k) -> float {
        const uint32_t lo = (uint32_t)bcast_i((int)(uint32_t)xr_ids, k);
        const uint32_t hi = (uint32_t)bcast_i((int)(uint32_t)(xr_ids >> 32), k);
        typedef const __attribute__((address_space(1))) char* global_bytes;      // device memory, not a flat address
        typedef const __attribute__((address_space(1))) float* global_float;
        const global_bytes row = (global_bytes)(uintptr_t)(((uint64_t)hi << 32) | lo);
        return *(global_float)(row + jj4);
    };
    // mu, inv_mu: m of the row just finished and 1 / it (the reference divides once per row, cpp:1329-1354:
    // here lane l does that division for the l-th row of a stretch, all 64 at once)
    float acc = 0.0f, run = 0.0f, mu = 1.0f, inv_mu = 1.0f;
    uint32_t p_cur = gidx[at(0)], p_nxt = gidx[at(kWave)];
    int2 i_cur = ginfo[at(0)], i_nxt = ginfo[at(kWave)];
    float f_cur = coef(p_cur), mr_cur = 1.0f, ir_cur = 1.0f;
    if constexpr (NORM) { mr_cur = m[i_cur.x]; ir_cur = 1.0f / mr_cur; }
    uint64_t xr_cur = x_row(p_cur), xr_nxt = x_row(p_nxt);
    float z[kWave];
#pragma unroll
    for (int k = 0; k < kWave; k++) z[k] = gather(xr_cur, k);
    for (int base = 0; base < count; base += kWave) {
        // requested first, needed last: the entries and rows of the stretch after the next, and what depends on
        // the next stretch's (their entries came in an iteration ago)
        const uint32_t p_far = gidx[at(base + 2 * kWave)];
        const int2 i_far = ginfo[at(base + 2 * kWave)];
        const float f_nxt = coef(p_nxt);
        float mr_nxt = 1.0f;
        if constexpr (NORM) mr_nxt = m[i_nxt.x];
        uint64_t yr_cur = (uint64_t)reinterpret_cast<uintptr_t>(Y) + (uint64_t)(uint32_t)i_cur.x * (uint64_t)ldy * 4u;
        int rs = 0;                                               // rows finished in this stretch (wave-uniform)
#pragma unroll
        for (int k = 0; k < kWave; k++) {
            // entries past the bin's last row (its padding) are added like any other: their sum is never stored
            acc = fmaf(bcast_f(f_cur, k), z[k], acc);
            z[k] = gather(xr_nxt, k);                                         // past the end: the last stretch again
            const uint32_t p = (uint32_t)bcast_i((int)p_cur, k);              // wave-uniform: the branch is scalar
            if (__builtin_expect((p & kStreamLast) != 0, 0)) {
                if (p & kStreamDummy) acc = 0.0f;                             // an empty row: its stand-in added nothing
                const int ctl = bcast_i(i_cur.y, rs);
                const int src = ctl & 63, dst = (ctl >> 8) & 63;
                const float mv = NORM ? bcast_f(mr_cur, rs) : 1.0f;
                if (src == CBM_WALK_LOAD_ONLY) {                              // a child of the root
                    run = NORM ? acc * mv : acc;
                } else {
                    float a = run, ma = mu, inv = inv_mu;
                    if (src) {
                        a = st[(src - 1) * kSlotFloats];
                        if constexpr (NORM) { ma = st[(src - 1) * kSlotFloats + kWave]; inv = st[(src - 1) * kSlotFloats + 2 * kWave]; }
                    }
                    if constexpr (NORM) {
                        if (all_body) run = fmaf(a, inv, acc) * mv;
                        else run = (jj < dv) ? fmaf(a, inv, acc) * mv : (acc + a / ma) * mv;
                    } else {
                        run = acc + a;
                    }
                }
                if (live) {
                    const uint32_t lo = (uint32_t)bcast_i((int)(uint32_t)yr_cur, rs);
                    const uint32_t hi = (uint32_t)bcast_i((int)(uint32_t)(yr_cur >> 32), rs);
                    typedef __attribute__((address_space(1))) char* global_bytes_out;
                    typedef __attribute__((address_space(1))) float* global_float_out;
                    const global_bytes_out row = (global_bytes_out)(uintptr_t)(((uint64_t)hi << 32) | lo);
                    *(global_float_out)(row + jj4) = (relu && run < 0.0f) ? 0.0f : run;   // keeps NaN, as torch.relu does
                }
                mu = mv;
                if constexpr (NORM) inv_mu = bcast_f(ir_cur, rs);
                if (dst) {
                    st[(dst - 1) * kSlotFloats] = run;
                    if constexpr (NORM) { st[(dst - 1) * kSlotFloats + kWave] = mv; st[(dst - 1) * kSlotFloats + 2 * kWave] = bcast_f(ir_cur, rs); }
                }
                acc = 0.0f;
                rs++;
            }
        }
        p_cur = p_nxt; p_nxt = p_far;
        i_cur = i_nxt; i_nxt = i_far;
        f_cur = f_nxt; mr_cur = mr_nxt;
        if constexpr (NORM) ir_cur = 1.0f / mr_cur;
        xr_nxt = x_row(p_far);
    }
}

// The walk of a SHALLOW tree in one launch, out of place: the wavefront of row v follows parent[]
// up to the child of the root above it (at most kMaxPathLevels - 1 steps, the ids kept one per
// lane), then adds the rows of Z down that path with exactly the arithmetic of propagate_row, so
// Y[v] comes out bit-identical to the level-by-level walk.  Every row recomputes the values of
// its ancestors instead of waiting for them: sum(depth) row reads instead of N, but no launch per
// level, and the ReLU can go into the store (no row is read back).  Z must not be Y: other
// wavefronts read the rows of Z while this one writes Y.
constexpr int kPathAhead = 4;              // rows of the path requested together

template <int VEC, int CH, bool NORM, bool FULL>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void propagate_paths(
    const int32_t* __restrict__ parent, const float* __restrict__ m, const float* __restrict__ Z,
    float* __restrict__ Y, int n, int d, int dv, int64_t ldz, int64_t ldy, int relu) {
    const int lane = threadIdx.x & (kWave - 1);
    const int v = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (v >= n) return;
    const int col0 = blockIdx.y * (kWave * VEC * CH) + lane * VEC;
    // lane t keeps the ancestor t steps above v (lane 0: v itself); k = steps to the child of the root
    int path = v, k = 0;
    for (int u = __builtin_amdgcn_readfirstlane(parent[v]); u >= 0 && k < kMaxPathLevels - 1;
         u = __builtin_amdgcn_readfirstlane(parent[u])) {
        k++;
        if (lane == k) path = u;
    }
    float my_m = 1.0f;
    if constexpr (NORM) if (lane <= k) my_m = m[path];
    float acc[CH][VEC];
    {
        const float* __restrict__ z = Z + (int64_t)bcast_i(path, k) * ldz + col0;
#pragma unroll
        for (int c = 0; c < CH; c++)
            if (FULL || col0 + c * kWave * VEC < d) load_vec<VEC>(z + c * kWave * VEC, acc[c]);
    }
    float mu = bcast_f(my_m, k);
    for (int t = k - 1; t >= 0; t -= kPathAhead) {
        float z[kPathAhead][CH][VEC];
#pragma unroll
        for (int a = 0; a < kPathAhead; a++) {             // past the end of the path: row v again, unused
            const float* __restrict__ zr = Z + (int64_t)bcast_i(path, max(t - a, 0)) * ldz + col0;
#pragma unroll
            for (int c = 0; c < CH; c++)
                if (FULL || col0 + c * kWave * VEC < d) load_vec<VEC>(zr + c * kWave * VEC, z[a][c]);
        }
#pragma unroll
        for (int a = 0; a < kPathAhead; a++)
            if (t - a >= 0) {
                const float mv = bcast_f(my_m, t - a);
                const float inv_mu = 1.0f / mu;
#pragma unroll
                for (int c = 0; c < CH; c++)
                    if (FULL || col0 + c * kWave * VEC < d) {
#pragma unroll
                        for (int e = 0; e < VEC; e++) {
                            if constexpr (NORM) {
                                const int j = col0 + c * kWave * VEC + e;
                                acc[c][e] = (j < dv) ? fmaf(acc[c][e], inv_mu, z[a][c][e]) * mv
                                                     : (z[a][c][e] + acc[c][e] / mu) * mv;
                            } else {
                                acc[c][e] = z[a][c][e] + acc[c][e];
                            }
                        }
                    }
                mu = mv;
            }
    }
    float* __restrict__ y = Y + (int64_t)v * ldy + col0;
#pragma unroll
    for (int c = 0; c < CH; c++)
        if (FULL || col0 + c * kWave * VEC < d) {
            if (relu) {
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[c][e] = acc[c][e] < 0.0f ? 0.0f : acc[c][e];   // keeps NaN
            }
            store_vec<VEC>(y + c * kWave * VEC, acc[c]);
        }
}

// Y[r,:] *= m[r] for the rows of level 0 (children of the root), cbm_extensions.cpp:910-940.
template <int VEC, int CH, bool FULL>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void scale_level0(
    const int32_t* __restrict__ order, int end, const float* __restrict__ m, float* __restrict__ Y, int d,
    int64_t ldy) {
    const int lane = threadIdx.x & (kWave - 1);
    const int i = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (i >= end) return;
    const int r = __builtin_amdgcn_readfirstlane(order[i]);
    const float s = m[r];
    const int col0 = blockIdx.y * (kWave * VEC * CH) + lane * VEC;
    float* __restrict__ y = Y + (int64_t)r * ldy + col0;
#pragma unroll
    for (int c = 0; c < CH; c++)
        if (FULL || col0 + c * kWave * VEC < d) {
            float t[VEC];
            load_vec<VEC>(y + c * kWave * VEC, t);
#pragma unroll
            for (int e = 0; e < VEC; e++) t[e] *= s;
            store_vec<VEC>(y + c * kWave * VEC, t);
        }
}

// Y = max(Y, 0) over an n x d matrix of row stride ldy: the ReLU of a multiply whose tree has more
// than one level (there the SpMM epilogue cannot apply it: children still need their parent's
// signed value).  One thread per element.
__global__ __launch_bounds__(256) void relu_rows(float* __restrict__ Y, int64_t total, int d, int64_t ldy) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    float* __restrict__ y = Y + (t / d) * ldy + (t % d);
    const float v = *y;
    if (v < 0.0f) *y = 0.0f;
}

// Rows that the schedule cut into pieces: Z[row] = (piece sums added in order, from 0) * scale,
// then the ReLU if asked.  long_rows = { row, first slot, pieces, bits(scale) } per cut row; a slot
// holds slot_floats floats, Z and d are those of the column range the slots cover.  One wavefront
// per cut row, lanes along the columns (VEC floats each).
template <int VEC>
__global__ __launch_bounds__(kWave * kWavesPerBlock) void combine_pieces(
    const int4* __restrict__ long_rows, const float* __restrict__ partials, float* __restrict__ Z, int n_long, int d,
    int64_t slot_floats, int64_t ldz, int apply_scale, int relu) {
    const int r = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (r >= n_long) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int4 lr = long_rows[r];
    const float scale = apply_scale ? __int_as_float(lr.w) : 1.0f;
    for (int j = lane * VEC; j < d; j += kWave * VEC) {
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = 0.0f;
        for (int k = 0; k < lr.z; k++) {
            float v[VEC];
            load_vec<VEC>(partials + (int64_t)(lr.y + k) * slot_floats + j, v);
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] += v[e];
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            acc[e] *= scale;
            if (relu) acc[e] = acc[e] < 0.0f ? 0.0f : acc[e];
        }
        store_vec<VEC>(Z + (int64_t)lr.x * ldz + j, acc);
    }
}

// ---------------------------------------------------------------------------------------------
// host side: shape selection and dispatch
// ---------------------------------------------------------------------------------------------
struct Tiling { int vec, ch, grid_y; bool full; };

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Largest vector width the alignment allows that still keeps 64 lanes busy; then as many
// 64-lane chunks per wave (1, 2 or 4) as d needs; anything wider is tiled over grid.y.
inline Tiling pick_tiling(int d, int64_t ld_a, int64_t ld_b, const void* pa, const void* pb) {
    int vmax = 1;
    if (d % 4 == 0 && ld_a % 4 == 0 && ld_b % 4 == 0 && aligned(pa, 16) && aligned(pb, 16)) vmax = 4;
    else if (d % 2 == 0 && ld_a % 2 == 0 && ld_b % 2 == 0 && aligned(pa, 8) && aligned(pb, 8)) vmax = 2;
    int vec = vmax;
    while (vec > 1 && d / vec < kWave) vec /= 2;
    const int units = (d + vec - 1) / vec;
    const int ch = units <= kWave ? 1 : (units <= 2 * kWave ? 2 : 4);
    const int tile = kWave * vec * ch;
    Tiling t;
    t.vec = vec; t.ch = ch; t.grid_y = (d + tile - 1) / tile; t.full = (d == t.grid_y * tile);
    return t;
}

// SpMM kernel choice: 0 = automatic, 1 = always one wave per row, 2 = slabs whenever the shape allows.
// A process-wide tuning hook; atomic so that threads launching on their own streams may read it
// while another thread sets it.
std::atomic<int> g_spmm_kernel{0};

// ---------------------------------------------------------------------------------------------
// (3) Row intersections for the builder: all pairs (i, j > i) of rows of A with
// 2 |row_i ^ row_j| > min(nnz_i, nnz_j) + alpha, the pairs the distance graph can admit
// (cbm_extensions.cpp:75-103; the reference gets |row_i ^ row_j| from mkl_sparse_syrk).
//
// One workgroup (16 wavefronts) per CU keeps `tile` 32-bit counters in LDS and takes rows from a
// shared ticket.  The candidate rows j are cut into tiles of `tile` consecutive ids; for every
// tile that can hold a j > i the workgroup walks, for every column c of row i, the rows j > i of
// that column (one wavefront per column, lanes along the column: coalesced; only the part of
// the sorted list that can hold ids of the tile, found by sampling the list with the 64 lanes)
// twice with a barrier in between:
//   1. increment counter j - tile start (LDS atomic);
//   2. swap the counter with 0 -- exactly one thread per distinct j gets the count, decides
//      admission and appends (i, j, s); the counters are clean for the next tile.
// Only the ticket and the output cursor are device-scope atomics.  Measured on 132 534 rows x
// 620 entries (25 G increments): 0.19 s (0.24 s when every tile re-read the whole lists); the
// same walks with the counters in device memory (workgroup-scope atomics executed by the L2)
// took 0.61-0.78 s; 16 host threads take 3.4 s.  What is left is the chain of dependent loads
// per (column, tile): column id -> list bounds -> samples -> list part.
// ---------------------------------------------------------------------------------------------
constexpr int kIsectWaves = 16;
constexpr int kIsectUnroll = 2;

// Part [beg, fin) of an ascending list of `len` row ids that can hold ids of the tile
// [lo_j, lo_j + tile): the 64 lanes sample the list at equal steps and two ballots bracket the
// tile's first and last element to within one step (ids outside the tile that fall into the
// bracket are filtered by the caller).  Wave-uniform result.
__device__ __forceinline__ void tile_range(const int32_t* __restrict__ lst, int len, int lo_j, int tile, int lane,
                                           int& beg, int& fin) {
    beg = 0; fin = 0;
    if (len <= 0) return;
    const int step = (len + kWave - 1) / kWave;
    const int at = lane * step;
    const int id = lst[min(at, len - 1)];
    const int below = __popcll(__ballot(at < len && id < lo_j));           // samples before the tile
    const int upto = __popcll(__ballot(at < len && id - lo_j < tile));      // samples before the tile's end
    beg = max(below - 1, 0) * step;
    fin = min(upto * step, len);
}

__global__ __launch_bounds__(kWave * kIsectWaves) void row_intersections(
    const int64_t* __restrict__ rowptr, const int32_t* __restrict__ col, const int64_t* __restrict__ colptr_t,
    const int32_t* __restrict__ row_t, const int64_t* __restrict__ after, const int32_t* __restrict__ row_nnz,
    int n, int alpha, int tile, uint32_t* __restrict__ ticket, cbm_pair* __restrict__ pairs,
    unsigned long long capacity, unsigned long long* __restrict__ n_pairs) {
    extern __shared__ uint32_t lds_cnt[];                    // `tile` counters
    __shared__ int s_row;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    for (int x = threadIdx.x; x < tile; x += kWave * kIsectWaves) lds_cnt[x] = 0u;
    for (;;) {
        __syncthreads();                                     // counters are zero; s_row may be overwritten
        if (threadIdx.x == 0) s_row = (int)atomicAdd(ticket, 1u);
        __syncthreads();
        const int i = s_row;
        if (i >= n) return;                                  // every thread of the workgroup sees the same ticket
        const int64_t b = rowptr[i], e = rowptr[i + 1];
        const int ni = row_nnz[i];
        for (int lo_j = ((i + 1) / tile) * tile; lo_j < n; lo_j += tile) {
            if (lo_j != ((i + 1) / tile) * tile) __syncthreads();          // previous tile's swaps are done
            // the bounds of the wave's next list are fetched while the current one is walked
            int64_t nx_a = 0, nx_hi = 0;
            if (b + wave < e) { nx_a = after[b + wave]; nx_hi = colptr_t[col[b + wave] + 1]; }
            for (int64_t k = b + wave; k < e; k += kIsectWaves) {
                const int32_t* __restrict__ lst = row_t + nx_a;
                const int len = (int)(nx_hi - nx_a);
                if (k + kIsectWaves < e) { nx_a = after[k + kIsectWaves]; nx_hi = colptr_t[col[k + kIsectWaves] + 1]; }
                int beg, fin;
                tile_range(lst, len, lo_j, tile, lane, beg, fin);
                for (int t0 = beg; t0 < fin; t0 += kWave * kIsectUnroll) {
                    int j[kIsectUnroll];
#pragma unroll
                    for (int u = 0; u < kIsectUnroll; u++) j[u] = lst[min(t0 + u * kWave + lane, fin - 1)];
#pragma unroll
                    for (int u = 0; u < kIsectUnroll; u++)
                        if (t0 + u * kWave + lane < fin && (unsigned)(j[u] - lo_j) < (unsigned)tile)
                            atomicAdd(&lds_cnt[j[u] - lo_j], 1u);
                }
            }
            __syncthreads();
            if (b + wave < e) { nx_a = after[b + wave]; nx_hi = colptr_t[col[b + wave] + 1]; }
            for (int64_t k = b + wave; k < e; k += kIsectWaves) {
                const int32_t* __restrict__ lst = row_t + nx_a;
                const int len = (int)(nx_hi - nx_a);
                if (k + kIsectWaves < e) { nx_a = after[k + kIsectWaves]; nx_hi = colptr_t[col[k + kIsectWaves] + 1]; }
                int beg, fin;
                tile_range(lst, len, lo_j, tile, lane, beg, fin);
                for (int t0 = beg; t0 < fin; t0 += kWave * kIsectUnroll) {   // whole wavefront iterates together (ballot below)
                    int j[kIsectUnroll];
#pragma unroll
                    for (int u = 0; u < kIsectUnroll; u++) j[u] = lst[min(t0 + u * kWave + lane, fin - 1)];
#pragma unroll
                    for (int u = 0; u < kIsectUnroll; u++) {
                        int sh = 0;
                        if (t0 + u * kWave + lane < fin && (unsigned)(j[u] - lo_j) < (unsigned)tile)
                            sh = (int)atomicExch(&lds_cnt[j[u] - lo_j], 0u);
                        // 2 s > min(n_i, n_j) + alpha; n_j is only fetched where n_i alone does not decide
                        bool keep = sh > 0;
                        if (keep && 2 * sh <= ni + alpha) keep = 2 * sh > row_nnz[j[u]] + alpha;
                        const unsigned long long mask = __ballot(keep);
                        if (mask) {
                            unsigned long long base = 0;
                            const int leader = __ffsll((long long)mask) - 1;
                            if (lane == leader) base = atomicAdd(n_pairs, (unsigned long long)__popcll(mask));
                            base = __shfl(base, leader, kWave);
                            if (keep) {
                                const unsigned long long at = base + __popcll(mask & ((1ull << lane) - 1ull));
                                if (at < capacity) pairs[at] = cbm_pair{i, j[u], sh};
                            }
                        }
                    }
                }
            }
        }
    }
}

// How a multiply of feature width d runs.
struct SlabPlan {
    int lpe = 0;            // lanes per delta entry: 8 -> 128-byte slabs, 16 -> 256-byte slabs, 0 -> one wave per row
    int n_slabs = 0;        // slabs the kernel walks (odd widths: padded count)
    bool relayout = false;  // the gather reads the slab-major copy in the workspace
    bool vec_out = false;   // rows of Z are float4-addressable
    int tail = 0;           // floats of the half slab behind the n_slabs full ones (copy only): 0 or 16
};

// Slabs of the slab-major copy: ceil(d / 32), rounded up to 1, 2, 4 or 8 when below 8 so that
// the XCDs sharing a slab split evenly.
inline int padded_slab_count(int d) {
    int ns = (d + 31) / 32;
    if (ns < kXcds) { int q = 1; while (q < ns) q *= 2; ns = q; }
    return ns;
}

// Layout of the slab-major copy of an n x d matrix: n_full slabs of 32 floats per row and, when
// the last d % 32 columns are at most 16, one half slab of 16 floats per row behind them (gathered
// with 4 lanes per entry, 16 entries per instruction: a width of 41 moves 48 floats per entry
// instead of 64).  The half slab is only taken where the full slabs still split evenly over the 8
// XCDs without padding (0, 1, 2, 4 or a multiple of 8 of them).
struct CopyLayout {
    int n_full = 0, tail = 0;                              // tail: 0 or 16 floats
    int64_t row_floats() const { return (int64_t)n_full * 32 + tail; }
};
inline CopyLayout copy_layout(int d) {
    CopyLayout c;
    const int nf = d / 32, rem = d % 32;
    const bool even_split = nf <= 2 || nf == 4 || nf % kXcds == 0;
    if (rem >= 1 && rem <= 16 && even_split) { c.n_full = nf; c.tail = 16; }
    else c.n_full = padded_slab_count(d);
    return c;
}
inline int64_t copy_floats(int64_t rows, int d) { return rows * copy_layout(d).row_floats(); }

// With a workspace every width runs on 128-byte slabs read from the slab-major copy (zero-padded
// for widths that are not a multiple of 32), unless the caller's row stride makes the copy
// pointless (below).  Without one, widths that split into whole 128- or
// 256-byte slabs whose count divides, or is a multiple of, the 8 XCDs gather from the row-major X
// (a 256-byte slab is taken when that still leaves one slab per XCD: d = 512, 1024, ...), and any
// other width or alignment takes one wavefront per row.  Measured at d = 512 / 1024 on an MI355X:
// 128-byte slabs from the copy beat 256-byte slabs from the row-major X by 5-18 % (copy included)
// on graphs with N >= 100 000 and tie on a 12 000-row graph.
// force_copy: the caller already made the copy.
inline SlabPlan plan_slabs(int d, int64_t ldx, int64_t ldz, const void* X, const void* Z, bool have_workspace,
                           bool force_copy) {
    SlabPlan p;
    if (g_spmm_kernel.load(std::memory_order_relaxed) == 1 && !force_copy) return p;
    const bool x_vec = d % 4 == 0 && ldx % 4 == 0 && aligned(X, 16);
    p.vec_out = d % 4 == 0 && ldz % 4 == 0 && aligned(Z, 16);
    SlabPlan direct;                                       // gather from the caller's row-major X
    if (d % 32 == 0 && x_vec && p.vec_out) {
        int lpe = 8;
        if (d % 64 == 0 && d / 64 >= kXcds) lpe = 16;
        const int ns = d / (lpe * 4);
        if (ns % kXcds == 0 || kXcds % ns == 0) { direct = p; direct.lpe = lpe; direct.n_slabs = ns; }
    }
    // A row stride of an odd number of 128-byte lines spreads the lines of a slab over all L2
    // channels by itself: the copy would buy nothing (100 000 x 256, 45 entries per row: 362 us
    // at a stride of 288 floats, 431 us at 256, 400 us with the copy).
    const bool alias_free = direct.lpe == 8 && ldx % 32 == 0 && (ldx / 32) % 2 == 1 && aligned(X, 128);
    if (force_copy || (have_workspace && !alias_free)) {
        const CopyLayout c = copy_layout(d);
        p.lpe = 8; p.n_slabs = c.n_full; p.tail = c.tail; p.relayout = true;
        return p;
    }
    return direct.lpe ? direct : p;
}

#define CBM_DISPATCH_TILING(T, LAUNCH)                                              \
    do {                                                                            \
        if ((T).full) { CBM_DISPATCH_VC(T, true, LAUNCH); }                         \
        else { CBM_DISPATCH_VC(T, false, LAUNCH); }                                 \
    } while (0)
#define CBM_DISPATCH_VC(T, FULLV, LAUNCH)                                           \
    do {                                                                            \
        switch ((T).vec * 10 + (T).ch) {                                            \
            case 11: LAUNCH(1, 1, FULLV); break;                                    \
            case 12: LAUNCH(1, 2, FULLV); break;                                    \
            case 14: LAUNCH(1, 4, FULLV); break;                                    \
            case 21: LAUNCH(2, 1, FULLV); break;                                    \
            case 22: LAUNCH(2, 2, FULLV); break;                                    \
            case 24: LAUNCH(2, 4, FULLV); break;                                    \
            case 41: LAUNCH(4, 1, FULLV); break;                                    \
            case 42: LAUNCH(4, 2, FULLV); break;                                    \
            default: LAUNCH(4, 4, FULLV); break;                                    \
        }                                                                           \
    } while (0)

inline int check_launch() { return hipGetLastError() == hipSuccess ? CBM_OK : CBM_ERR_LAUNCH; }

inline int check_matrix(int32_t n, int32_t d, int64_t ld) {
    if (n < 0 || d < 0 || ld < d) return CBM_ERR_SHAPE;
    return CBM_OK;
}

// Wavefronts per SIMD the persistent slab kernel is launched with (a workgroup is one wavefront on
// each of a CU's 4 SIMDs).  Every wavefront keeps 8 KB of gathered lines in flight while it is inside
// a long row; at the 6-7 wavefronts the registers allow, a 32-CU XCD has more lines in flight than
// its 4 MB L2 holds.  Short rows spend more of their time outside the gather rounds and need the
// extra wavefronts.  Measured on an MI355X with 128-byte slabs: rows averaging 190-490 entries are
// fastest at 3-4 (3-8 % over 6-8), rows averaging 45 entries at 5-6 (4 costs 7 %, 3 costs 20 %),
// rows averaging 13 entries at the register limit (6 costs 7 %); 256-byte slabs are fastest at
// 3-4 on every graph tried.
std::atomic<int> g_spmm_occupancy{0};                      // 0 = automatic
// Tiled multiply: 1 = the kernel of the local blocks gathers the remote entries too (when no row is
// cut), 0 = the remote entries always go through the slab kernel first.  A tuning hook.
std::atomic<int> g_tiled_fused{1};
inline int slab_waves_per_simd(int64_t nnz, int32_t n, int lpe) {
    const int fixed = g_spmm_occupancy.load(std::memory_order_relaxed);
    if (fixed > 0) return fixed;
    if (lpe == 16) return 4;
    // long rows: 4 where a slab of X (n x 128 bytes) exceeds an XCD's 4 MB L2, 6 where it stays resident
    // (12,000 rows of 194 entries, d = 128: 77.8 us at 4, 74.1 us at 6; 2 costs 29 %)
    if (nnz >= (int64_t)128 * n) return (int64_t)n * 128 <= ((int64_t)4 << 20) ? 6 : 4;
    return nnz >= (int64_t)32 * n ? 6 : 8;                 // 8: every wavefront the registers allow
}

// Per-device launch facts of the persistent slab kernel, queried once per device (a process may
// drive several devices from several threads): compute units, and for every instantiation the
// workgroups per XCD that are resident at once.
constexpr int kMaxDevices = 64;
struct DeviceFacts {
    int cus = 0;
    int groups[2][3][3] = {};                              // [PACKED][lpe: 8, 16, 4][coefficient mode]
};
DeviceFacts g_facts[kMaxDevices];
std::atomic<int> g_facts_ready[kMaxDevices];               // zero-initialised
std::mutex g_facts_mutex;

template <class K>
int resident_groups_per_xcd(K kernel, int cus) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kWave * kWavesPerBlock, 0) != hipSuccess) return 0;
    if (cus < kXcds || per_cu < 1) return 0;
    return (cus / kXcds) * per_cu;
}

constexpr int kTailRounds = 4;                             // 4 lanes per entry: 16 entries per instruction, 64 per round

template <bool PACKED>
void fill_groups(int (&g)[3][3], int cus) {
    g[2][kCoefStream] = resident_groups_per_xcd(spmm_slab_per_xcd<4, PACKED, kCoefStream, kTailRounds>, cus);
    g[2][kCoefSign] = resident_groups_per_xcd(spmm_slab_per_xcd<4, PACKED, kCoefSign, kTailRounds>, cus);
    g[2][kCoefSignM] = resident_groups_per_xcd(spmm_slab_per_xcd<4, PACKED, kCoefSignM, kTailRounds>, cus);
    g[0][kCoefStream] = resident_groups_per_xcd(spmm_slab_per_xcd<8, PACKED, kCoefStream, CBM_SLAB_ROUNDS>, cus);
    g[0][kCoefSign] = resident_groups_per_xcd(spmm_slab_per_xcd<8, PACKED, kCoefSign, CBM_SLAB_ROUNDS>, cus);
    g[0][kCoefSignM] = resident_groups_per_xcd(spmm_slab_per_xcd<8, PACKED, kCoefSignM, CBM_SLAB_ROUNDS>, cus);
    g[1][kCoefStream] = resident_groups_per_xcd(spmm_slab_per_xcd<16, PACKED, kCoefStream, CBM_SLAB_ROUNDS>, cus);
    g[1][kCoefSign] = resident_groups_per_xcd(spmm_slab_per_xcd<16, PACKED, kCoefSign, CBM_SLAB_ROUNDS>, cus);
    g[1][kCoefSignM] = resident_groups_per_xcd(spmm_slab_per_xcd<16, PACKED, kCoefSignM, CBM_SLAB_ROUNDS>, cus);
}

// Facts of the CURRENT device, or nullptr if they cannot be had.
const DeviceFacts* device_facts() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    if (!g_facts_ready[dev].load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_facts_mutex);
        if (!g_facts_ready[dev].load(std::memory_order_relaxed)) {
            DeviceFacts f;
            if (hipDeviceGetAttribute(&f.cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return nullptr;
            fill_groups<false>(f.groups[0], f.cus);
            fill_groups<true>(f.groups[1], f.cus);
            g_facts[dev] = f;
            g_facts_ready[dev].store(1, std::memory_order_release);
        }
    }
    return &g_facts[dev];
}

// Byte ranges [a, a + bytes_a) and [b, b + bytes_b) share at least one byte.
inline bool ranges_overlap(const void* a, int64_t bytes_a, const void* b, int64_t bytes_b) {
    const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return bytes_a > 0 && bytes_b > 0 && pa < pb + (uintptr_t)bytes_b && pb < pa + (uintptr_t)bytes_a;
}
inline int64_t matrix_bytes(int32_t n, int32_t d, int64_t ld) {
    return n > 0 && d > 0 ? ((int64_t)(n - 1) * ld + d) * 4 : 0;
}

inline int launch_relayout(const float* X, float* workspace, int32_t n, int32_t d, int64_t ldx, hipStream_t s,
                           const float* mask = nullptr, int64_t ldm = 0, const float* scale = nullptr) {
    const CopyLayout c = copy_layout(d);
    const int ns = c.n_full, tail4 = c.tail / 4;
    const int64_t blocks = ((int64_t)n * (ns * 8 + tail4) + 255) / 256;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    const dim3 grid((unsigned)blocks), block(256);
    const bool vec = d % 4 == 0 && ldx % 4 == 0 && aligned(X, 16) && (!mask || (ldm % 4 == 0 && aligned(mask, 16)));
#define LAUNCH_RELAYOUT(V, K, S) \
    hipLaunchKernelGGL((relayout_slabs<V, K, S>), grid, block, 0, s, X, workspace, n, d, ns, tail4, ldx, mask, ldm, scale)
    switch ((vec ? 4 : 0) | (mask ? 2 : 0) | (scale ? 1 : 0)) {
        case 0: LAUNCH_RELAYOUT(false, false, false); break;
        case 1: LAUNCH_RELAYOUT(false, false, true); break;
        case 2: LAUNCH_RELAYOUT(false, true, false); break;
        case 3: LAUNCH_RELAYOUT(false, true, true); break;
        case 4: LAUNCH_RELAYOUT(true, false, false); break;
        case 5: LAUNCH_RELAYOUT(true, false, true); break;
        case 6: LAUNCH_RELAYOUT(true, true, false); break;
        default: LAUNCH_RELAYOUT(true, true, true); break;
    }
#undef LAUNCH_RELAYOUT
    return CBM_OK;
}

// n_desc / partials: a schedule that cuts long rows has n_desc >= n descriptors and needs the scratch
// area for the piece sums (slab kernel only); n_desc = 0 means one descriptor per row.
template <bool PACKED>
int launch_spmm(const int32_t* rowptr, const uint32_t* idx, int64_t nnz, const float* val, const float* m,
                const int32_t* parent, const int32_t* sched, const float* X, float* Z, float* workspace,
                int32_t flags, int32_t n, int32_t d, int64_t ldx, int64_t ldz, hipStream_t s, int32_t n_desc = 0,
                float* partials = nullptr, int32_t n_pieces = 0) {
    if (flags & ~(CBM_SPMM_WORKSPACE_READY | CBM_SPMM_RELU | CBM_SPMM_WORKSPACE_PRESCALED | CBM_SPMM_SCHED_BATCHED))
        return CBM_ERR_UNSUPPORTED;
    const int relu = (flags & CBM_SPMM_RELU) ? 1 : 0;
    // a batched schedule: n + 1 descriptors; rows cut into pieces have their own kind of schedule
    const int batched = (flags & CBM_SPMM_SCHED_BATCHED) ? 1 : 0;
    if (batched && (!sched || n_desc > 0)) return CBM_ERR_UNSUPPORTED;
    if ((flags & CBM_SPMM_WORKSPACE_PRESCALED) && (!PACKED || !m || !(flags & CBM_SPMM_WORKSPACE_READY)))
        return CBM_ERR_UNSUPPORTED;                       // only a ready copy of a normalised multiply can be pre-scaled
    if ((!rowptr && !sched) || !X || !Z) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (int rc = check_matrix(n, d, ldz)) return rc;
    if (sched && !aligned(sched, 16)) return CBM_ERR_SHAPE;
    // rows of X are gathered while rows of Z are written: the two must not share a byte
    if (X == Z || ranges_overlap(X, matrix_bytes(n, d, ldx), Z, matrix_bytes(n, d, ldz))) return CBM_ERR_SHAPE;
    const bool ready = (flags & CBM_SPMM_WORKSPACE_READY) != 0;
    if (workspace) {                                      // the slab-major copy must be disjoint from X and Z
        if (!aligned(workspace, 16)) return CBM_ERR_SHAPE;
        const int64_t ws_bytes = copy_floats(n, d) * 4;
        if (ranges_overlap(workspace, ws_bytes, X, matrix_bytes(n, d, ldx)) ||
            ranges_overlap(workspace, ws_bytes, Z, matrix_bytes(n, d, ldz)))
            return CBM_ERR_SHAPE;
    }
    const bool have_ws = workspace != nullptr;
    if (ready && !have_ws) return CBM_ERR_NULL;
    if (n == 0 || d == 0) return CBM_OK;
    const int4* sc = reinterpret_cast<const int4*>(sched);
    const SlabPlan plan = plan_slabs(d, ldx, ldz, X, Z, have_ws, ready);
    if (plan.lpe) {
        const int lpe = plan.lpe, n_slabs = plan.n_slabs;
        const float* Xg = X;                              // what the gather reads
        int64_t x_slab_stride = lpe * 4, x_row_stride = ldx;
        // A normalised multiply that copies X anyway scales row c of the copy by m[c]: the entries
        // then need no coefficient at all, only their sign (4 bytes per entry and slab less to stream).
        bool prescaled = (flags & CBM_SPMM_WORKSPACE_PRESCALED) != 0;
        if (plan.relayout) {
            if (!ready) {
                prescaled = PACKED && m != nullptr;
                if (int rc = launch_relayout(X, workspace, n, d, ldx, s, nullptr, 0, prescaled ? m : nullptr)) return rc;
            }
            Xg = workspace; x_slab_stride = (int64_t)n * lpe * 4; x_row_stride = lpe * 4;
        }
        const int coef_mode = prescaled ? kCoefSign : (val ? kCoefStream : (m ? kCoefSignM : kCoefSign));
        const DeviceFacts* facts = device_facts();
        const int per_wave = facts ? facts->cus / kXcds : 0;
        const int n_rows = n_desc > 0 ? n_desc : n;             // descriptors the waves walk
        // One launch over `slabs` slabs of `L` float4 per row: the full slabs, then (copy only) the half slab
        // of the last d % 32 columns as a launch of its own with 4 lanes per entry.
        auto launch = [&](int L, int slabs, const float* Xl, int64_t slab_stride, int64_t row_stride, float* Zl, int d_l,
                          float* partials_l) -> int {
            int G = facts ? facts->groups[PACKED ? 1 : 0][L == 8 ? 0 : (L == 16 ? 1 : 2)][coef_mode] : 0;
            if (G <= 0) return CBM_ERR_LAUNCH;
            const int cap = per_wave * slab_waves_per_simd(nnz, n, L);
            if (cap > 0 && G > cap) G = cap;
            // no more waves than rows: with fewer rows than resident waves shrink the grid
            const int share = slabs >= kXcds ? 1 : kXcds / slabs;
            const int need = (n_rows + share * kWavesPerBlock - 1) / (share * kWavesPerBlock);
            if (G > need) G = need;
            const dim3 grid(G * kXcds), block(kWave * kWavesPerBlock);
            const int vec_out = (plan.vec_out && aligned(Zl, 16)) ? 1 : 0;
#define LAUNCH_SLAB(LL, CF, UU)                                                                                  \
    hipLaunchKernelGGL((spmm_slab_per_xcd<LL, PACKED, CF, UU>), grid, block, 0, s, rowptr, sc, idx, val, m, parent, \
                       Xl, Zl, n_rows, d_l, vec_out, slabs, slab_stride, row_stride, ldz, relu, partials_l,             \
                       (batched && nnz > 0) ? 1 : 0)
            switch (L * 4 + coef_mode) {
                case 8 * 4 + kCoefStream: LAUNCH_SLAB(8, kCoefStream, CBM_SLAB_ROUNDS); break;
                case 8 * 4 + kCoefSign: LAUNCH_SLAB(8, kCoefSign, CBM_SLAB_ROUNDS); break;
                case 8 * 4 + kCoefSignM: LAUNCH_SLAB(8, kCoefSignM, CBM_SLAB_ROUNDS); break;
                case 16 * 4 + kCoefStream: LAUNCH_SLAB(16, kCoefStream, CBM_SLAB_ROUNDS); break;
                case 16 * 4 + kCoefSign: LAUNCH_SLAB(16, kCoefSign, CBM_SLAB_ROUNDS); break;
                case 16 * 4 + kCoefSignM: LAUNCH_SLAB(16, kCoefSignM, CBM_SLAB_ROUNDS); break;
                case 4 * 4 + kCoefStream: LAUNCH_SLAB(4, kCoefStream, kTailRounds); break;
                case 4 * 4 + kCoefSign: LAUNCH_SLAB(4, kCoefSign, kTailRounds); break;
                default: LAUNCH_SLAB(4, kCoefSignM, kTailRounds); break;
            }
#undef LAUNCH_SLAB
            return CBM_OK;
        };
        int rc = CBM_OK;
        if (n_slabs > 0)
            rc = launch(lpe, n_slabs, Xg, x_slab_stride, x_row_stride, Z, plan.tail ? n_slabs * 32 : d, partials);
        if (rc == CBM_OK && plan.tail)                        // partials of the tail: behind those of the full slabs
            rc = launch(4, 1, workspace + (int64_t)n * n_slabs * 32, 0, plan.tail, Z + n_slabs * 32, d - n_slabs * 32,
                        partials ? partials + (int64_t)n_pieces * n_slabs * 32 : nullptr);
        if (rc == CBM_OK) return check_launch();
        if (ready) return CBM_ERR_LAUNCH;                 // no occupancy information: cannot honour the copy
    }
    if (n_desc > 0) return CBM_ERR_UNSUPPORTED;           // a cut schedule runs on the slab kernel only
    const Tiling t = pick_tiling(d, ldx, ldz, X, Z);
    const dim3 grid((n + kWavesPerBlock - 1) / kWavesPerBlock, t.grid_y), block(kWave * kWavesPerBlock);
#define LAUNCH(V, C, F)                                                                              \
    hipLaunchKernelGGL((spmm_wave_per_row<V, C, PACKED, F>), grid, block, 0, s, rowptr, idx, val, m, \
                       parent, sc, X, Z, n, d, ldx, ldz, relu)
    CBM_DISPATCH_TILING(t, LAUNCH);
#undef LAUNCH
    return check_launch();
}

template <bool NORM>
int launch_propagate(const int32_t* parent, const int32_t* order, const int32_t* level_off_dev,
                     const int32_t* lo, int32_t n_levels, const float* m, float* Y, int32_t n, int32_t d,
                     int64_t ldy, int32_t flags, hipStream_t s) {
    // n_levels may be a prefix of the tree's levels: the subtree walk takes over below it
    const Tiling t = pick_tiling(d, ldy, ldy, Y, Y);
    const int dv = d - d % 8;
    const dim3 block(kWave * kWavesPerBlock);
    if (NORM && (flags & CBM_PROP_SCALE_ROOTS) && lo[1] > lo[0]) {
        const dim3 grid((lo[1] + kWavesPerBlock - 1) / kWavesPerBlock, t.grid_y);
#define LAUNCH(V, C, F) \
    hipLaunchKernelGGL((scale_level0<V, C, F>), grid, block, 0, s, order, lo[1], m, Y, d, ldy)
        CBM_DISPATCH_TILING(t, LAUNCH);
#undef LAUNCH
    }
    int l = 1;
    while (l < n_levels) {
        const int width = lo[l + 1] - lo[l];
        auto chain_end = [&](int from) {                   // end of the run of single-row levels at `from`
            int e = from;
            while (e < n_levels && lo[e + 1] - lo[e] == 1) e++;
            return e;
        };
        if (width == 1) {                                  // a chain of single-row levels
            const int l_end = chain_end(l);
            if (l_end - l >= kMinChain) {
                const int waves = (d + kWave - 1) / kWave;
                const int wpb = waves < kNarrowWaves ? waves : kNarrowWaves;
                const dim3 grid((waves + wpb - 1) / wpb), cblock(kWave * wpb);
                hipLaunchKernelGGL((propagate_chain<NORM>), grid, cblock, 0, s, parent, order, lo[l], l_end - l, m, Y,
                                   d, dv, ldy);
                l = l_end;
                continue;
            }
        }
        if (width <= kNarrowWidth) {
            int l_end = l + 1;                             // extend over narrow levels, but leave chains to the chain kernel
            while (l_end < n_levels && lo[l_end + 1] - lo[l_end] <= kNarrowWidth &&
                   chain_end(l_end) - l_end < kMinChain) l_end++;
            if (l_end - l >= 2) {
                const dim3 grid(1, t.grid_y), nblock(kWave * kNarrowWaves);
#define LAUNCH(V, C, F)                                                                                 \
    hipLaunchKernelGGL((propagate_narrow_levels<V, C, NORM, F>), grid, nblock, 0, s, parent, order,     \
                       level_off_dev, l, l_end, m, Y, d, dv, ldy)
                CBM_DISPATCH_TILING(t, LAUNCH);
#undef LAUNCH
                l = l_end;
                continue;
            }
        }
        const dim3 grid((width + kWavesPerBlock - 1) / kWavesPerBlock, t.grid_y);
#define LAUNCH(V, C, F)                                                                                 \
    hipLaunchKernelGGL((propagate_level<V, C, NORM, F>), grid, block, 0, s, parent, order, lo[l],       \
                       lo[l + 1], m, Y, d, dv, ldy)
        CBM_DISPATCH_TILING(t, LAUNCH);
#undef LAUNCH
        l++;
    }
    return check_launch();
}

int validate_levels(const int32_t* lo, int32_t n_levels, int32_t n) {
    if (n_levels < 0) return CBM_ERR_SHAPE;
    if (n_levels == 0) return n == 0 ? CBM_OK : CBM_ERR_SHAPE;
    if (lo[0] != 0 || lo[n_levels] != n) return CBM_ERR_SHAPE;
    for (int l = 0; l < n_levels; l++)
        if (lo[l + 1] < lo[l]) return CBM_ERR_SHAPE;
    return CBM_OK;
}

// ---------------------------------------------------------------------------------------------
// Static scratch of cbm_spmm_update_static_f32, the entry point that allocates nothing: the
// slab-major copy of X lives in this array instead of a workspace the caller brings.  Every
// device the library runs on holds its own copy of the array (CBM_STATIC_SCRATCH_FLOATS floats)
// at its own address until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and copies get the per-device address looked up below.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) float scratch[CBM_STATIC_SCRATCH_FLOATS];

float* g_scratch_ptr[kMaxDevices];                         // device address of `scratch`, per device
std::atomic<int> g_scratch_ready[kMaxDevices];             // zero-initialised
std::mutex g_scratch_mutex;

// Address of the CURRENT device's copy of `scratch`, looked up once per device.
int static_scratch(float** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return CBM_ERR_LAUNCH;
    if (dev < 0 || dev >= kMaxDevices) return CBM_ERR_UNSUPPORTED;
    if (!g_scratch_ready[dev].load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ready[dev].load(std::memory_order_relaxed)) {
            void* ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
                (void)hipGetLastError();
                return CBM_ERR_LAUNCH;
            }
            g_scratch_ptr[dev] = static_cast<float*>(ptr);
            g_scratch_ready[dev].store(1, std::memory_order_release);
        }
    }
    *out = g_scratch_ptr[dev];
    return CBM_OK;
}

template <bool NORM>
int launch_subtrees(const cbm_walk_dev* w, const float* m, float* Y, int32_t d, int64_t ldy, hipStream_t s) {
    if (w->n_bins == 0) return CBM_OK;
    const int slices = (d + kWave - 1) / kWave;
    const int64_t waves = (int64_t)w->n_bins * slices;
    const int64_t blocks = (waves + kSubWaves - 1) / kSubWaves;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    const size_t lds = (size_t)kSubWaves * w->n_slots * kSlotFloats * sizeof(float);     // at most 93 KB
    hipLaunchKernelGGL((propagate_subtrees<NORM>), dim3((unsigned)blocks), dim3(kWave * kSubWaves), lds, s,
                       reinterpret_cast<const int2*>(w->entries), w->bin_off, w->n_bins, slices, m, Y, d, d - d % 8, ldy,
                       w->n_slots);
    return check_launch();
}

template <bool NORM>
int launch_stream(const cbm_walk_stream_dev* w, const float* m, const float* X, float* Y, int32_t d, int64_t ldx,
                  int64_t ldy, int relu, hipStream_t s) {
    if (w->n_bins == 0) return CBM_OK;
    const int slices = (d + kWave - 1) / kWave;
    const int64_t waves = (int64_t)w->n_bins * slices;
    const int64_t blocks = (waves + kSubWaves - 1) / kSubWaves;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    const size_t lds = (size_t)kSubWaves * w->n_slots * kSlotFloats * sizeof(float);     // at most 93 KB
    hipLaunchKernelGGL((spmm_update_subtrees<NORM>), dim3((unsigned)blocks), dim3(kWave * kSubWaves), lds, s, w->gidx,
                       reinterpret_cast<const int2*>(w->ginfo), w->bin_goff, w->n_bins, slices, m, X, Y, d, d - d % 8, ldx,
                       ldy, w->n_slots, relu);
    return check_launch();
}

}  // namespace

extern "C" {

const char* cbm_version(void) { return "cbm4gnn_amd hip 0.1 (gfx950)"; }

const char* cbm_status_string(int status) {
    switch (status) {
        case CBM_OK: return "ok";
        case CBM_ERR_NULL: return "a required pointer is NULL";
        case CBM_ERR_ALLOC: return "allocation failed";
        case CBM_ERR_SHAPE: return "size, stride or index out of range";
        case CBM_ERR_LAUNCH: return "HIP launch failed";
        case CBM_ERR_INTERNAL: return "internal invariant failed";
        case CBM_ERR_UNSUPPORTED: return "not implemented in this build";
        case CBM_ERR_SCRATCH: return "shape needs more scratch than the static array holds (CBM_STATIC_SCRATCH_FLOATS)";
        default: return "unknown status";
    }
}

int cbm_spmm_f32(const int32_t* rowptr, const uint32_t* idx, int64_t nnz, const float* m, const float* coef,
                 const int32_t* parent, const int32_t* row_sched, const float* X, float* Z, float* workspace,
                 int32_t flags, int32_t n, int32_t d, int64_t ldx, int64_t ldz, void* stream) {
    if (!idx && n > 0) return CBM_ERR_NULL;
    if (coef && !m) return CBM_ERR_NULL;                 // coef is the expansion of m, not a substitute
    return launch_spmm<true>(rowptr, idx, nnz, coef, m, parent, row_sched, X, Z, workspace, flags, n, d, ldx, ldz,
                             static_cast<hipStream_t>(stream));
}

int cbm_relayout_slabs_f32(const float* X, float* workspace, int32_t n, int32_t d, int64_t ldx, void* stream) {
    if (!X || !workspace) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (!aligned(workspace, 16) || X == workspace) return CBM_ERR_SHAPE;
    if (n == 0 || d == 0) return CBM_OK;
    if (int rc = launch_relayout(X, workspace, n, d, ldx, static_cast<hipStream_t>(stream))) return rc;
    return check_launch();
}

int cbm_relayout_slabs_scaled_f32(const float* X, const float* scale, float* workspace, int32_t n, int32_t d, int64_t ldx,
                                  void* stream) {
    if (!X || !workspace || !scale) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (!aligned(workspace, 16)) return CBM_ERR_SHAPE;
    if (ranges_overlap(workspace, copy_floats(n, d) * 4, X, matrix_bytes(n, d, ldx))) return CBM_ERR_SHAPE;
    if (n == 0 || d == 0) return CBM_OK;
    if (int rc = launch_relayout(X, workspace, n, d, ldx, static_cast<hipStream_t>(stream), nullptr, 0, scale)) return rc;
    return check_launch();
}

int cbm_relayout_slabs_masked_f32(const float* X, const float* mask, const float* scale, float* workspace, int32_t n,
                                  int32_t d, int64_t ldx, int64_t ldm, void* stream) {
    if (!X || !workspace || !mask) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (int rc = check_matrix(n, d, ldm)) return rc;
    if (!aligned(workspace, 16)) return CBM_ERR_SHAPE;
    const int64_t ws_bytes = copy_floats(n, d) * 4;
    if (ranges_overlap(workspace, ws_bytes, X, matrix_bytes(n, d, ldx)) ||
        ranges_overlap(workspace, ws_bytes, mask, matrix_bytes(n, d, ldm)))
        return CBM_ERR_SHAPE;
    if (n == 0 || d == 0) return CBM_OK;
    if (int rc = launch_relayout(X, workspace, n, d, ldx, static_cast<hipStream_t>(stream), mask, ldm, scale)) return rc;
    return check_launch();
}

int64_t cbm_relayout_floats(int32_t n, int32_t d) {
    if (n <= 0 || d <= 0) return 0;
    return copy_floats(n, d);
}

int cbm_row_intersections_groups(void) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return cus;                                            // the LDS allocation allows one workgroup per CU
}

int cbm_row_intersections(const int64_t* rowptr, const int32_t* col, const int64_t* colptr_t, const int32_t* row_t,
                          const int64_t* after, const int32_t* row_nnz, int32_t n, int32_t alpha, int32_t groups,
                          uint32_t* ticket, cbm_pair* pairs, int64_t capacity, unsigned long long* n_pairs,
                          void* stream) {
    if (n < 0 || capacity < 0 || groups < 0) return CBM_ERR_SHAPE;
    if (n == 0) return CBM_OK;
    if (!rowptr || !col || !colptr_t || !row_t || !after || !row_nnz || !ticket || !n_pairs) return CBM_ERR_NULL;
    if (capacity > 0 && !pairs) return CBM_ERR_NULL;
    if (groups < 1) return CBM_ERR_SHAPE;
    int dev = 0, lds = 0;
    if (hipGetDevice(&dev) != hipSuccess) return CBM_ERR_LAUNCH;
    if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return CBM_ERR_LAUNCH;
    int tile = 1 << 15;                                    // 128 KB of counters where the device allows it
    while (tile > 1024 && (int64_t)tile * 4 + 1024 > lds) tile >>= 1;
    while (tile > 1024 && tile / 2 >= n) tile >>= 1;       // small matrices: no larger than needed
    const size_t bytes = (size_t)tile * 4;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(row_intersections), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)bytes) != hipSuccess)
        return CBM_ERR_LAUNCH;
    hipLaunchKernelGGL(row_intersections, dim3((unsigned)groups), dim3(kWave * kIsectWaves), bytes,
                       static_cast<hipStream_t>(stream), rowptr, col, colptr_t, row_t, after, row_nnz, n, alpha, tile,
                       ticket, pairs, (unsigned long long)capacity, n_pairs);
    return check_launch();
}

int cbm_set_spmm_occupancy(int waves_per_simd) {
    if (waves_per_simd < 0 || waves_per_simd > 8) return CBM_ERR_SHAPE;
    g_spmm_occupancy = waves_per_simd;
    return CBM_OK;
}

int cbm_set_spmm_kernel(int kind) {
    if (kind < 0 || kind > 2) return CBM_ERR_SHAPE;
    g_spmm_kernel = kind;
    return CBM_OK;
}

int cbm_spmm_summation_groups(int32_t d, int64_t ldx, int64_t ldz, const void* X, const void* Z, int32_t have_workspace) {
    const SlabPlan p = plan_slabs(d, ldx, ldz, X, Z, have_workspace != 0, false);
    if (!p.lpe) return 1;
    return p.n_slabs > 0 ? kWave / p.lpe : kWave / 4;      // only the half slab: d <= 16
}

int cbm_set_tiled_fused(int on) {
    g_tiled_fused.store(on ? 1 : 0, std::memory_order_relaxed);
    return CBM_OK;
}

int cbm_spmm_tail_columns(int32_t d, int64_t ldx, int64_t ldz, const void* X, const void* Z, int32_t have_workspace) {
    const SlabPlan p = plan_slabs(d, ldx, ldz, X, Z, have_workspace != 0, false);
    return (p.lpe && p.tail) ? d - p.n_slabs * 32 : 0;
}

int64_t cbm_spmm_workspace_floats(int32_t n, int32_t d, int64_t ldx, int64_t ldz, const void* X, const void* Z) {
    if (n <= 0 || d <= 0) return 0;
    const SlabPlan p = plan_slabs(d, ldx, ldz, X, Z, true, false);
    return p.relayout ? copy_floats(n, d) : 0;
}

int cbm_expand_coef_f32(const uint32_t* idx, const float* m, float* coef, int64_t nnz, void* stream) {
    if (nnz < 0) return CBM_ERR_SHAPE;
    if (nnz == 0) return CBM_OK;
    if (!idx || !m || !coef) return CBM_ERR_NULL;
    const int64_t blocks = (nnz + 255) / 256;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    hipLaunchKernelGGL(expand_coef, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), idx, m,
                       coef, nnz);
    return check_launch();
}

int csr_spmm_f32(const int32_t* rowptr, const int32_t* col, int64_t nnz, const float* val, const int32_t* row_sched,
                 const float* X, float* Y, float* workspace, int32_t flags, int32_t n, int32_t d, int64_t ldx,
                 int64_t ldy, void* stream) {
    if (!col && n > 0) return CBM_ERR_NULL;
    return launch_spmm<false>(rowptr, reinterpret_cast<const uint32_t*>(col), nnz, val, nullptr, nullptr, row_sched,
                              X, Y, workspace, flags, n, d, ldx, ldy, static_cast<hipStream_t>(stream));
}

int cbm_propagate_f32(const int32_t* parent, const int32_t* order, const int32_t* level_off_dev,
                      const int32_t* level_off_host, int32_t n_levels, const float* m, float* Y, int32_t n,
                      int32_t d, int64_t ldy, int32_t flags, void* stream) {
    if (!parent || !order || !level_off_dev || !level_off_host || !Y) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldy)) return rc;
    if (int rc = validate_levels(level_off_host, n_levels, n)) return rc;
    if (flags & ~CBM_PROP_SCALE_ROOTS) return CBM_ERR_UNSUPPORTED;
    if (n == 0 || d == 0) return CBM_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return m ? launch_propagate<true>(parent, order, level_off_dev, level_off_host, n_levels, m, Y, n, d, ldy, flags, s)
             : launch_propagate<false>(parent, order, level_off_dev, level_off_host, n_levels, m, Y, n, d, ldy, flags, s);
}

int cbm_propagate_subtrees_f32(const cbm_walk_dev* walk, const int32_t* parent, const int32_t* order,
                               const int32_t* level_off_dev, const int32_t* level_off_host, int32_t n_levels, const float* m,
                               float* Y, int32_t n, int32_t d, int64_t ldy, int32_t flags, void* stream) {
    if (!walk || !parent || !order || !level_off_dev || !level_off_host || !Y) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldy)) return rc;
    if (int rc = validate_levels(level_off_host, n_levels, n)) return rc;
    if (flags & ~(CBM_PROP_SCALE_ROOTS | CBM_UPDATE_RELU)) return CBM_ERR_UNSUPPORTED;
    if (n == 0 || d == 0) return CBM_OK;
    if (walk->cut < 0 || walk->cut >= n_levels || walk->n_bins < 0 || walk->n_entries < 0 || walk->n_slots < 0 ||
        walk->n_slots > CBM_WALK_MAX_SLOTS)
        return CBM_ERR_SHAPE;
    if (walk->n_bins > 0 && (!walk->entries || !walk->bin_off || !aligned(walk->entries, 8))) return CBM_ERR_NULL;
    if ((int64_t)n * ldy * 4 > ((int64_t)1 << 46)) return CBM_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // levels 1 .. cut level by level (and the scale of the root's children, if asked), then every subtree below
    const int32_t prop_flags = flags & CBM_PROP_SCALE_ROOTS;
    int rc = m ? launch_propagate<true>(parent, order, level_off_dev, level_off_host, walk->cut + 1, m, Y, n, d, ldy, prop_flags, s)
               : launch_propagate<false>(parent, order, level_off_dev, level_off_host, walk->cut + 1, m, Y, n, d, ldy, prop_flags, s);
    if (rc) return rc;
    rc = m ? launch_subtrees<true>(walk, m, Y, d, ldy, s) : launch_subtrees<false>(walk, m, Y, d, ldy, s);
    if (rc || !(flags & CBM_UPDATE_RELU)) return rc;
    const int64_t total = (int64_t)n * d, blocks = (total + 255) / 256;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    hipLaunchKernelGGL(relu_rows, dim3((unsigned)blocks), dim3(256), 0, s, Y, total, d, ldy);
    return check_launch();
}

int cbm_spmm_update_subtrees_f32(const cbm_walk_stream_dev* ws, const float* m, const float* X, float* Y, int32_t n,
                                 int32_t d, int64_t ldx, int64_t ldy, int32_t flags, void* stream) {
    if (!ws || !X || !Y) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (int rc = check_matrix(n, d, ldy)) return rc;
    if (flags & ~CBM_UPDATE_RELU) return CBM_ERR_UNSUPPORTED;
    if (X == Y) return CBM_ERR_SHAPE;                    // rows of Y are stored while rows of X are still gathered
    if (n == 0 || d == 0) return CBM_OK;
    if (ws->n != n || ws->n_bins < 0 || ws->n_elems < 0 || ws->n_elems % kWave != 0 || ws->n_slots < 0 ||
        ws->n_slots > CBM_WALK_MAX_SLOTS || (int64_t)ws->n_bins * kWave > ws->n_elems)
        return CBM_ERR_SHAPE;                            // bins are whole stretches of 64 entries
    if ((uint32_t)n > kStreamCol) return CBM_ERR_SHAPE;  // the column shares its word with two flags and the sign
    if (ws->n_bins > 0 && (!ws->gidx || !ws->ginfo || !ws->bin_goff || !aligned(ws->ginfo, 8))) return CBM_ERR_NULL;
    if ((int64_t)n * ldy * 4 > ((int64_t)1 << 46) || (int64_t)n * ldx * 4 > ((int64_t)1 << 46)) return CBM_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int relu = (flags & CBM_UPDATE_RELU) != 0;
    return m ? launch_stream<true>(ws, m, X, Y, d, ldx, ldy, relu, s) : launch_stream<false>(ws, m, X, Y, d, ldx, ldy, relu, s);
}

int cbm_spmm_update_f32(const int32_t* rowptr, const uint32_t* idx, int64_t nnz, const float* m, const float* coef,
                        const int32_t* parent, const int32_t* row_sched, const int32_t* order, const int32_t* level_off_dev,
                        const int32_t* level_off_host, int32_t n_levels, const float* X, float* Y, float* workspace,
                        int32_t n, int32_t d, int64_t ldx, int64_t ldy, int32_t flags, void* stream) {
    if (!parent) return CBM_ERR_NULL;
    if (flags & ~(CBM_PROP_SCALE_ROOTS | CBM_UPDATE_RELU | CBM_UPDATE_WORKSPACE_READY | CBM_UPDATE_WORKSPACE_PRESCALED |
                  CBM_UPDATE_SCHED_BATCHED))
        return CBM_ERR_UNSUPPORTED;
    if (X == Y) return CBM_ERR_SHAPE;                    // the SpMM overwrites Y while gathering X
    const bool relu = (flags & CBM_UPDATE_RELU) != 0;
    // With a flat tree the SpMM's store is the final value of every row: the ReLU goes into its
    // epilogue.  With deeper trees rows must keep their signed value for their children, so the
    // ReLU is a pass of its own after the walk.
    const bool flat = n_levels <= 1;
    int spmm_flags = (flags & CBM_UPDATE_WORKSPACE_READY) ? CBM_SPMM_WORKSPACE_READY : 0;
    if (flags & CBM_UPDATE_WORKSPACE_PRESCALED) spmm_flags |= CBM_SPMM_WORKSPACE_PRESCALED;
    if (flags & CBM_UPDATE_SCHED_BATCHED) spmm_flags |= CBM_SPMM_SCHED_BATCHED;
    if (relu && flat) spmm_flags |= CBM_SPMM_RELU;
    int rc = cbm_spmm_f32(rowptr, idx, nnz, m, coef, parent, row_sched, X, Y, workspace, spmm_flags, n, d, ldx, ldy,
                          stream);
    if (rc) return rc;
    // children of the root were scaled by the SpMM epilogue already
    rc = cbm_propagate_f32(parent, order, level_off_dev, level_off_host, n_levels, m, Y, n, d, ldy, 0, stream);
    if (rc || !relu || flat || n == 0 || d == 0) return rc;
    const int64_t total = (int64_t)n * d, blocks = (total + 255) / 256;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    hipLaunchKernelGGL(relu_rows, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), Y, total, d, ldy);
    return check_launch();
}

int cbm_spmm_update_paths_f32(const int32_t* rowptr, const uint32_t* idx, int64_t nnz, const float* m, const float* coef,
                              const int32_t* parent, const int32_t* row_sched, const int32_t* order,
                              const int32_t* level_off_dev, const int32_t* level_off_host, int32_t n_levels, const float* X,
                              float* Y, float* workspace, float* z_scratch, int32_t n, int32_t d, int64_t ldx, int64_t ldy,
                              int32_t flags, void* stream) {
    if (n_levels < 2 || n_levels > kMaxPathLevels || n <= 0 || d <= 0)     // flat or deep: the level plan
        return cbm_spmm_update_f32(rowptr, idx, nnz, m, coef, parent, row_sched, order, level_off_dev, level_off_host,
                                   n_levels, X, Y, workspace, n, d, ldx, ldy, flags, stream);
    if (!parent || !z_scratch || !Y) return CBM_ERR_NULL;
    if (X == Y) return CBM_ERR_SHAPE;                    // as cbm_spmm_update_f32
    if (flags & ~(CBM_PROP_SCALE_ROOTS | CBM_UPDATE_RELU | CBM_UPDATE_WORKSPACE_READY | CBM_UPDATE_WORKSPACE_PRESCALED |
                  CBM_UPDATE_SCHED_BATCHED))
        return CBM_ERR_UNSUPPORTED;
    if (int rc = check_matrix(n, d, ldy)) return rc;
    if (int rc = validate_levels(level_off_host, n_levels, n)) return rc;
    if (!aligned(z_scratch, 16)) return CBM_ERR_SHAPE;
    const int64_t ldz = (d + 3) & ~3;                     // rows of the scratch start on 16 bytes
    const int64_t z_bytes = (int64_t)n * ldz * 4;
    if (ranges_overlap(z_scratch, z_bytes, Y, matrix_bytes(n, d, ldy)) ||
        ranges_overlap(z_scratch, z_bytes, X, matrix_bytes(n, d, ldx)) ||
        (workspace && ranges_overlap(z_scratch, z_bytes, workspace, copy_floats(n, d) * 4)))
        return CBM_ERR_SHAPE;
    int spmm_flags = (flags & CBM_UPDATE_WORKSPACE_READY) ? CBM_SPMM_WORKSPACE_READY : 0;
    if (flags & CBM_UPDATE_WORKSPACE_PRESCALED) spmm_flags |= CBM_SPMM_WORKSPACE_PRESCALED;
    if (flags & CBM_UPDATE_SCHED_BATCHED) spmm_flags |= CBM_SPMM_SCHED_BATCHED;
    // children of the root are scaled by the SpMM epilogue: their rows of the scratch are final
    if (int rc = cbm_spmm_f32(rowptr, idx, nnz, m, coef, parent, row_sched, X, z_scratch, workspace, spmm_flags, n, d, ldx,
                              ldz, stream))
        return rc;
    const Tiling t = pick_tiling(d, ldz, ldy, z_scratch, Y);
    const dim3 grid((n + kWavesPerBlock - 1) / kWavesPerBlock, t.grid_y), block(kWave * kWavesPerBlock);
    const int dv = d - d % 8, relu = (flags & CBM_UPDATE_RELU) ? 1 : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define LAUNCH(V, C, F)                                                                                         \
    do {                                                                                                        \
        if (m) hipLaunchKernelGGL((propagate_paths<V, C, true, F>), grid, block, 0, s, parent, m, z_scratch, Y, \
                                  n, d, dv, ldz, ldy, relu);                                                    \
        else hipLaunchKernelGGL((propagate_paths<V, C, false, F>), grid, block, 0, s, parent, m, z_scratch, Y,  \
                                n, d, dv, ldz, ldy, relu);                                                      \
    } while (0)
    CBM_DISPATCH_TILING(t, LAUNCH);
#undef LAUNCH
    return check_launch();
}

int cbm_spmm_update_single_f32(const int32_t* rowptr, const uint32_t* idx, const float* m, const float* coef,
                               const int32_t* parent, int32_t n_levels, const float* X, float* Y, int32_t n, int32_t d,
                               int64_t ldx, int64_t ldy, int32_t flags, void* stream) {
    if (flags & ~(CBM_PROP_SCALE_ROOTS | CBM_UPDATE_RELU)) return CBM_ERR_UNSUPPORTED;
    if (n_levels < 0 || n_levels > kMaxPathLevels) return CBM_ERR_UNSUPPORTED;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (int rc = check_matrix(n, d, ldy)) return rc;
    if (n == 0 || d == 0) return CBM_OK;
    if (!rowptr || !parent || !X || !Y || (!idx && n > 0)) return CBM_ERR_NULL;
    if (X == Y || ranges_overlap(X, matrix_bytes(n, d, ldx), Y, matrix_bytes(n, d, ldy))) return CBM_ERR_SHAPE;
    const Tiling t = pick_tiling(d, ldx, ldy, X, Y);
    const dim3 grid((n + kWavesPerBlock - 1) / kWavesPerBlock, t.grid_y), block(kWave * kWavesPerBlock);
    const int dv = d - d % 8, relu = (flags & CBM_UPDATE_RELU) ? 1 : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define LAUNCH(V, C, F)                                                                                              \
    do {                                                                                                             \
        if (m) hipLaunchKernelGGL((spmm_update_paths_wave_per_row<V, C, true, F>), grid, block, 0, s, rowptr, idx,   \
                                  coef, m, parent, X, Y, n, d, dv, ldx, ldy, relu);                                  \
        else hipLaunchKernelGGL((spmm_update_paths_wave_per_row<V, C, false, F>), grid, block, 0, s, rowptr, idx,    \
                                nullptr, m, parent, X, Y, n, d, dv, ldx, ldy, relu);                                 \
    } while (0)
    CBM_DISPATCH_TILING(t, LAUNCH);
#undef LAUNCH
    return check_launch();
}

int64_t cbm_spmm_update_paths_scratch_floats(int32_t n, int32_t d, int32_t n_levels) {
    if (n <= 0 || d <= 0 || n_levels < 2 || n_levels > kMaxPathLevels) return 0;
    return (int64_t)n * ((d + 3) & ~3);
}

int64_t cbm_spmm_tiled_workspace_floats(const cbm_tiling_dev* t, int32_t n, int32_t d) {
    if (!t || n <= 0 || d <= 0) return 0;
    return copy_floats((int64_t)n + (t->n_long > 0 ? t->n_pieces : 0), d);
}

int cbm_spmm_tiled_f32(const cbm_tiling_dev* t, const float* m, const float* X, float* Z, float* workspace, int32_t flags,
                       int32_t n, int32_t d, int64_t ldx, int64_t ldz, void* stream) {
    if (!t || !X || !Z || !workspace) return CBM_ERR_NULL;
    if (t->n_long < 0 || t->n_pieces < 0 || t->n_sched_r < 0) return CBM_ERR_SHAPE;
    if (t->n_long > 0 && (!t->long_rows || !t->sched_r || t->n_sched_r < n || !aligned(t->long_rows, 16))) return CBM_ERR_NULL;
    if (t->n_long == 0 && t->n_sched_r != 0 && t->n_sched_r != n) return CBM_ERR_SHAPE;
    if (!t->panel_ptr || !t->rowptr_r || (t->n_blocks > 0 && (!t->blk_tile || !t->seg || !t->lidx))) return CBM_ERR_NULL;
    if (t->nnz_remote > 0 && !t->idx_r) return CBM_ERR_NULL;
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (int rc = check_matrix(n, d, ldz)) return rc;
    if (t->tile_rows != 1024 && t->tile_rows != 512) return CBM_ERR_SHAPE;
    if (t->n_panels != (n + kPanelRows - 1) / kPanelRows || t->n_blocks < 0) return CBM_ERR_SHAPE;
    if (flags & ~(CBM_SPMM_WORKSPACE_READY | CBM_SPMM_RELU | CBM_SPMM_WORKSPACE_PRESCALED)) return CBM_ERR_UNSUPPORTED;
    const bool ready = (flags & CBM_SPMM_WORKSPACE_READY) != 0;
    // the local entries carry no coefficient: with m, the copy they gather from must be the scaled one
    if (ready && ((m != nullptr) != ((flags & CBM_SPMM_WORKSPACE_PRESCALED) != 0))) return CBM_ERR_UNSUPPORTED;
    if (!ready && (flags & CBM_SPMM_WORKSPACE_PRESCALED)) return CBM_ERR_UNSUPPORTED;
    if (n == 0 || d == 0) return CBM_OK;
    // as cbm_spmm_f32: X and Z must not share a byte, nor the workspace with either
    if (X == Z || ranges_overlap(X, matrix_bytes(n, d, ldx), Z, matrix_bytes(n, d, ldz))) return CBM_ERR_SHAPE;
    if (!aligned(workspace, 16)) return CBM_ERR_SHAPE;
    {
        const int64_t ws_bytes = cbm_spmm_tiled_workspace_floats(t, n, d) * 4;
        if (ranges_overlap(workspace, ws_bytes, X, matrix_bytes(n, d, ldx)) ||
            ranges_overlap(workspace, ws_bytes, Z, matrix_bytes(n, d, ldz)))
            return CBM_ERR_SHAPE;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const DeviceFacts* facts = device_facts();
    if (!facts || facts->cus < kXcds) return CBM_ERR_LAUNCH;
    if (!ready) {
        if (int rc = launch_relayout(X, workspace, n, d, ldx, s, nullptr, 0, m)) return rc;
    }
    // remote entries: the slab kernel from the copy.  With local blocks the left scale and the ReLU
    // wait for the kernel of the local part; without any, this launch (and the combine pass for cut
    // rows) is the whole multiply and applies them.
    const bool has_local = t->n_blocks > 0;
    const int relu = (flags & CBM_SPMM_RELU) ? 1 : 0;
    const CopyLayout lay = copy_layout(d);
    const int n_full = lay.n_full, d_full = lay.tail ? n_full * 32 : d, d_tail = lay.tail ? d - n_full * 32 : 0;
    float* partials = t->n_long > 0 ? workspace + copy_floats(n, d) : nullptr;
    const int remote_flags = CBM_SPMM_WORKSPACE_READY | (m ? CBM_SPMM_WORKSPACE_PRESCALED : 0) |
                             ((relu && !has_local) ? CBM_SPMM_RELU : 0);
    // With local blocks and no cut rows, the kernel of the local part gathers the remote entries too.
    const bool fused = has_local && t->n_long == 0 && (int64_t)n * 128 < ((int64_t)1 << 32) &&
                       g_tiled_fused.load(std::memory_order_relaxed) != 0;
    if (!fused)
        if (int rc = launch_spmm<true>(t->rowptr_r, t->idx_r, t->nnz_remote, nullptr, m, nullptr, t->sched_r, X, Z, workspace,
                                       remote_flags, n, d, ldx, ldz, s, t->n_long > 0 ? t->n_sched_r : 0, partials,
                                       t->n_pieces))
            return rc;
    if (t->n_long > 0) {                                  // pieces of cut rows -> their rows of Z, per column range
        const int4* lr = reinterpret_cast<const int4*>(t->long_rows);
        const int scale_here = has_local ? 0 : 1, relu_here = (relu && !has_local) ? 1 : 0;
        const dim3 cgrid((unsigned)((t->n_long + kWavesPerBlock - 1) / kWavesPerBlock)), cblock(kWave * kWavesPerBlock);
        if (n_full > 0) {
            // slots are whole slabs (a multiple of 32 floats, 16-byte aligned): float4 where Z allows it
            if (d_full % 4 == 0 && ldz % 4 == 0 && aligned(Z, 16))
                hipLaunchKernelGGL(combine_pieces<4>, cgrid, cblock, 0, s, lr, partials, Z, t->n_long, d_full,
                                   (int64_t)n_full * 32, ldz, scale_here, relu_here);
            else
                hipLaunchKernelGGL(combine_pieces<1>, cgrid, cblock, 0, s, lr, partials, Z, t->n_long, d_full,
                                   (int64_t)n_full * 32, ldz, scale_here, relu_here);
        }
        if (lay.tail)
            hipLaunchKernelGGL(combine_pieces<1>, cgrid, cblock, 0, s, lr, partials + (int64_t)t->n_pieces * n_full * 32,
                               Z + n_full * 32, t->n_long, d_tail, (int64_t)lay.tail, ldz, scale_here, relu_here);
    }
    if (!has_local) return check_launch();
    // local entries: tiles of the copy staged in LDS; adds to Z, then scale and ReLU
    const int G = facts->cus / kXcds;                     // 129 KB of LDS: one workgroup per CU
#define LAUNCH_TILED_F(T, S, L, F, WL, ZL, DL, SLABS)                                                                    \
    do {                                                                                                                 \
        const size_t bytes_ = (size_t)(T + 1) * L * 16;                                                                  \
        const int vec_ = (d % 4 == 0 && ldz % 4 == 0 && aligned(ZL, 16)) ? 1 : 0;                                        \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(spmm_tiled_local<T, S, L, F>),                             \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes_) != hipSuccess)                  \
            return CBM_ERR_LAUNCH;                                                                                       \
        hipLaunchKernelGGL((spmm_tiled_local<T, S, L, F>), dim3(G * kXcds), dim3(kWave * kTiledWaves), bytes_, s,        \
                           t->panel_ptr, t->blk_tile, t->seg, t->lidx, t->rowptr_r, t->idx_r, WL, ZL, t->row_scale, n,   \
                           DL, SLABS, t->n_panels, ldz, relu, vec_);                                                     \
    } while (0)
#define LAUNCH_TILED(T, S, L, WL, ZL, DL, SLABS)                                                                         \
    do {                                                                                                                 \
        if (fused) LAUNCH_TILED_F(T, S, L, true, WL, ZL, DL, SLABS);                                                     \
        else LAUNCH_TILED_F(T, S, L, false, WL, ZL, DL, SLABS);                                                          \
    } while (0)
#define LAUNCH_TILED_BOTH(T, S)                                                                                          \
    do {                                                                                                                 \
        if (n_full > 0) LAUNCH_TILED(T, S, 8, workspace, Z, d_full, n_full);                                             \
        if (lay.tail) LAUNCH_TILED(T, S, 4, workspace + (int64_t)n * n_full * 32, Z + n_full * 32, d_tail, 1);          \
    } while (0)
    if (t->tile_rows == 1024) { if (t->has_negative) LAUNCH_TILED_BOTH(1024, true); else LAUNCH_TILED_BOTH(1024, false); }
    else { if (t->has_negative) LAUNCH_TILED_BOTH(512, true); else LAUNCH_TILED_BOTH(512, false); }
#undef LAUNCH_TILED_BOTH
#undef LAUNCH_TILED
#undef LAUNCH_TILED_F
    return check_launch();
}

int cbm_spmm_update_tiled_f32(const cbm_tiling_dev* t, const float* m, const int32_t* parent, const int32_t* order,
                              const int32_t* level_off_dev, const int32_t* level_off_host, int32_t n_levels,
                              const float* X, float* Y, float* workspace, int32_t n, int32_t d, int64_t ldx, int64_t ldy,
                              int32_t flags, void* stream) {
    if (!parent) return CBM_ERR_NULL;
    if (flags & ~(CBM_PROP_SCALE_ROOTS | CBM_UPDATE_RELU | CBM_UPDATE_WORKSPACE_READY | CBM_UPDATE_WORKSPACE_PRESCALED))
        return CBM_ERR_UNSUPPORTED;
    const bool relu = (flags & CBM_UPDATE_RELU) != 0;
    const bool flat = n_levels <= 1;
    int spmm_flags = (flags & CBM_UPDATE_WORKSPACE_READY) ? CBM_SPMM_WORKSPACE_READY : 0;
    if (flags & CBM_UPDATE_WORKSPACE_PRESCALED) spmm_flags |= CBM_SPMM_WORKSPACE_PRESCALED;
    if (relu && flat) spmm_flags |= CBM_SPMM_RELU;
    int rc = cbm_spmm_tiled_f32(t, m, X, Y, workspace, spmm_flags, n, d, ldx, ldy, stream);
    if (rc) return rc;
    rc = cbm_propagate_f32(parent, order, level_off_dev, level_off_host, n_levels, m, Y, n, d, ldy, 0, stream);
    if (rc || !relu || flat || n == 0 || d == 0) return rc;
    const int64_t total = (int64_t)n * d, blocks = (total + 255) / 256;
    if (blocks > INT32_MAX) return CBM_ERR_SHAPE;
    hipLaunchKernelGGL(relu_rows, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), Y, total, d, ldy);
    return check_launch();
}

int cbm_spmm_update_static_f32(const int32_t* rowptr, const uint32_t* idx, int64_t nnz, const float* m,
                               const float* coef, const int32_t* parent, const int32_t* row_sched,
                               const int32_t* order, const int32_t* level_off_dev, const int32_t* level_off_host,
                               int32_t n_levels, const float* X, float* Y, int32_t n, int32_t d, int64_t ldx,
                               int64_t ldy, int32_t flags, void* stream) {
    if (int rc = check_matrix(n, d, ldx)) return rc;
    if (int rc = check_matrix(n, d, ldy)) return rc;
    if (flags & (CBM_UPDATE_WORKSPACE_READY | CBM_UPDATE_WORKSPACE_PRESCALED))
        return CBM_ERR_UNSUPPORTED;                       // the scratch is not the caller's to fill
    const int64_t need = cbm_spmm_workspace_floats(n, d, ldx, ldy, X, Y);
    if (need > (int64_t)CBM_STATIC_SCRATCH_FLOATS) return CBM_ERR_SCRATCH;
    float* ws = nullptr;                                  // need == 0: this shape gathers from X in place
    if (need > 0)
        if (int rc = static_scratch(&ws)) return rc;
    // relayout_slabs overwrites every float of the copy it makes (padding columns included), so
    // nothing of the previous call's contents has to be cleared.
    return cbm_spmm_update_f32(rowptr, idx, nnz, m, coef, parent, row_sched, order, level_off_dev, level_off_host,
                               n_levels, X, Y, ws, n, d, ldx, ldy, flags, stream);
}

}  // extern "C"
