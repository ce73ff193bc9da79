// dense^T x dense -> block-sparse (weight gradient on the sparse support):
//   out[32b + j][i] = sum_t G[t][32r + i] * X[t][32c + j]   for every data block b at (r, c).
//
// One workgroup owns an SR x SC rectangle of block positions of W and one slice of the tokens.
// It lists the nonzero blocks inside its rectangle from the CSR arrays, deals them out to its
// waves (at most QW accumulators each; more blocks than that are done in further passes), and
// streams the tokens in chunks of TC: the chunk's G[TC, 32*SR] and X[TC, 32*SC] panels are
// staged in LDS once, double buffered through registers, and shared by all blocks of the tile.
// With more than one token slice the fp32 partial blocks go to a workspace and a second kernel
// adds them in slice order, so the result does not depend on scheduling.
#pragma once
#include "pbs_common.h"

namespace pbs {

struct SddArgs {
    const void* g;           // [M, N] grad_output, row-major
    const void* x;           // [M, K] input, row-major
    const int32_t* ptr;      // row_start_ends_a [N/32 + 1]
    const int32_t* idx;      // cols_a [nnz][2] = (block col, data block)
    void* out;               // [nnz*32, 32] (T) when nsplit == 1
    float* partial;          // [nsplit][nnz*1024] fp32 when nsplit > 1
    int M, N, K, nnz;
    int tiles_r, tiles_c, nsplit;
    int tokens_per_split;    // multiple of TC
    int segs;                // segment kernel: equal shares of a row band's blocks (tiles_c is unused there)
};

// Which block rows of W form row band `band` of rectangles (SR places; -1 = no row).  Normally they are
// rows SR*band .. SR*band + SR - 1.  When the per-row block counts are very uneven (largest > 2x the
// mean) the rows are ranked by count and dealt to the bands in serpentine order, so that all
// rectangles hold about the same number of blocks.  Every workgroup derives its own band from the
// row pointer array (a few microseconds at most; above SDD_BALANCE_MAX_ROWS rows the natural order
// is kept).  Called by all threads of the workgroup; `scratch` is LDS for nblk_r + 2 ints.  Returns
// whether the row pointers were scanned; then s_ptr_copy (if given, nblk_r + 1 ints of LDS) holds them.
constexpr int SDD_BALANCE_MAX_ROWS = 1024;
static __device__ __forceinline__ bool sdd_band_rows(const int32_t* __restrict__ ptr, int nnz, int nblk_r, int tiles_r, int band,
                                                     int SR, int* s_rowid, int* scratch, int tid, int nthreads,
                                                     int* s_ptr_copy = nullptr, int rows_per_band = 0) {
    if (rows_per_band <= 0 || rows_per_band > SR) rows_per_band = SR;   // natural order: rows band * rows_per_band ...
    bool skewed = false;
    const bool scanned = nblk_r <= SDD_BALANCE_MAX_ROWS && tiles_r >= 2;
    if (scanned) {
        int* s_max = scratch + nblk_r;
        int* s_sum = s_max + 1;
        if (tid == 0) {
            *s_max = 0;
            *s_sum = 0;
        }
        __syncthreads();
        for (int r = tid; r < nblk_r; r += nthreads) {
            const int lo = clamp_entry(ptr[r], nnz), hi = clamp_entry(ptr[r + 1], nnz);
            const int n = hi > lo ? hi - lo : 0;
            if (s_ptr_copy) {   // saves the caller a second trip to global memory
                s_ptr_copy[r] = lo;
                if (r == nblk_r - 1) s_ptr_copy[nblk_r] = hi;
            }
            scratch[r] = n;
            atomicMax(s_max, n);
            atomicAdd(s_sum, n);
        }
        __syncthreads();
        skewed = (long long)*s_max * nblk_r > 2ll * *s_sum;
    }
    if (tid < SR) {
        const int r = band * rows_per_band + tid;
        s_rowid[tid] = (!skewed && tid < rows_per_band && r < nblk_r) ? r : -1;
    }
    __syncthreads();
    if (skewed) {
        for (int r = tid; r < nblk_r; r += nthreads) {
            const int n = scratch[r];
            int rank = 0;
            for (int o = 0; o < nblk_r; ++o) {
                const int m = scratch[o];
                rank += (m > n || (m == n && o < r)) ? 1 : 0;
            }
            const int place = rank / tiles_r;
            int b = rank % tiles_r;
            if (place & 1) b = tiles_r - 1 - b;
            if (b == band && place < SR) s_rowid[place] = r;
        }
        __syncthreads();
    }
    return scanned;
}

template <typename T, int SR, int SC, int QW, int NW>
struct SddCfg {
    using E = Elem<T>;
    static constexpr int NT = NW * 64;
    static constexpr int TC = (E::ESZ == 4) ? 16 : 32;     // tokens per staged chunk
    static constexpr int FG = SR * 32;                      // features per token row, G panel
    static constexpr int FX = SC * 32;
    // fp32: [t][f] words.  bf16: token pairs interleaved, [t/2][f] words of (t even, t odd).
    static constexpr int ROWS = (E::ESZ == 4) ? TC : TC / 2;
    static constexpr int G_BYTES = ROWS * FG * 4;
    static constexpr int X_BYTES = ROWS * FX * 4;
    static constexpr int STAGE_BYTES = G_BYTES + X_BYTES;
    static constexpr int CG = TC * FG * E::ESZ / 16;        // 16-byte chunks per chunk of tokens
    static constexpr int CX = TC * FX * E::ESZ / 16;
    static constexpr int NG = CG / NT;
    static constexpr int NX = CX / NT;
    static constexpr int QMAX = QW * NW;
    static constexpr int LIST_MAX = SR * SC;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES + (LIST_MAX + SR + 4) * 4;
    static_assert(CG % NT == 0 && CX % NT == 0, "staging must divide evenly");
    static_assert(E::ESZ == 4 || (NG % 2 == 0 && NX % 2 == 0), "bf16 stages token pairs");
    static_assert(SR <= 64 && SC <= 255 && SR <= 255, "list entry packs (rl, cl) in bytes");
};

template <typename T, int SR, int SC, int QW, int NW>
__global__ __launch_bounds__(NW * 64) void sdd_kernel(SddArgs a) {
    using C = SddCfg<T, SR, SC, QW, NW>;
    using E = typename C::E;
    constexpr int NT = C::NT, TC = C::TC, FG = C::FG, FX = C::FX;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* stage0 = smem;
    int* s_list = reinterpret_cast<int*>(smem + 2 * C::STAGE_BYTES);  // (b << 12) | (rl << 8)... see pack
    int* s_blk = s_list;                                               // [LIST_MAX] data block id
    // the (rl, cl) pair of each listed block lives in a second array to keep ids full width
    __shared__ unsigned short s_pos[C::LIST_MAX];
    int* s_rowoff = s_list + C::LIST_MAX;                              // [SR+1]
    __shared__ int s_count;

    const int ntiles = a.tiles_r * a.tiles_c;
    const int wg = xcd_tile_id(blockIdx.x, ntiles * a.nsplit);
    if (wg < 0) return;
    const int sp = wg / ntiles;            // token slice: slices of one tile land on different XCDs
    const int tile = wg % ntiles;
    const int tr = tile / a.tiles_c;
    const int tc = tile % a.tiles_c;
    const int c0 = tc * SC;
    const int nblk_r = a.N / 32;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lrow = lane & 31;
    const int h = lane >> 5;

    // ---- list the nonzero blocks of the rectangle, row-major ----
    int my_lo = 0, my_n = 0;
    __shared__ int s_rowid[SR];   // block row of W in each place of this rectangle's band, or -1
    sdd_band_rows(a.ptr, a.nnz, nblk_r, a.tiles_r, tr, SR, s_rowid, reinterpret_cast<int*>(smem), tid, NT);
    if (tid < SR) {
        const int r = s_rowid[tid];
        if (r >= 0) {
            const int lo = clamp_entry(a.ptr[r], a.nnz), hi = clamp_entry(a.ptr[r + 1], a.nnz);
            // rows are sorted by block column: first entry with column >= c0
            int l = lo, u = hi;
            while (l < u) {
                const int mid = (l + u) >> 1;
                if (a.idx[2 * mid] < c0) l = mid + 1; else u = mid;
            }
            my_lo = l;
            while (l < hi && a.idx[2 * l] < c0 + SC) ++l;
            my_n = l - my_lo;
            if (my_n > SC) my_n = SC;   // (a list with repeated columns: never more entries than the tables hold)
        }
        s_rowoff[tid] = my_n;
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int i = 0; i < SR; ++i) {
            const int n = s_rowoff[i];
            s_rowoff[i] = run;
            run += n;
        }
        s_rowoff[SR] = run;
        s_count = run;
    }
    __syncthreads();
    if (tid < SR) {
        const int off = s_rowoff[tid];
        for (int i = 0; i < my_n; ++i) {
            const int c = a.idx[2 * (my_lo + i)];
            int b = a.idx[2 * (my_lo + i) + 1];
            if (b < 0 || b >= a.nnz) b = -1;
            s_blk[off + i] = b;
            s_pos[off + i] = (unsigned short)((tid << 8) | (c - c0));
        }
    }
    __syncthreads();
    const int nq = s_count;
    if (nq == 0) return;

    const int t_begin = sp * a.tokens_per_split;
    int t_end = t_begin + a.tokens_per_split;
    if (t_end > a.M) t_end = a.M;
    const int nchunks = t_begin < t_end ? (t_end - t_begin + TC - 1) / TC : 0;

    const unsigned char* G = static_cast<const unsigned char*>(a.g);
    const unsigned char* X = static_cast<const unsigned char*>(a.x);
    const size_t x_col0 = (size_t)c0 * 32 * E::ESZ;
    const int x_valid = (a.K - c0 * 32) * E::ESZ;
    // byte offset, inside a G row, of the 16-byte piece at panel byte cb (-1: that block row does not exist)
    auto g_piece = [&](int cb) -> int {
        const int rid = s_rowid[cb / (32 * E::ESZ)];
        return rid < 0 ? -1 : rid * 32 * E::ESZ + cb % (32 * E::ESZ);
    };

    uint4 rg[C::NG];
    uint4 rx[C::NX];

    // one 16-byte chunk of a panel: token row `t`, byte offset `cb` inside the panel's row
    auto ld_panel = [&](const unsigned char* base, size_t ld_bytes, size_t col0, int valid, int t, int cb) -> uint4 {
        if (t < t_end && cb < valid) return ldg16(base + (size_t)t * ld_bytes + col0 + cb);
        return make_uint4(0, 0, 0, 0);
    };
    auto ld_g = [&](size_t ld_bytes, int t, int piece) -> uint4 {
        if (t < t_end && piece >= 0) return ldg16(G + (size_t)t * ld_bytes + piece);
        return make_uint4(0, 0, 0, 0);
    };
    // the G pieces a thread stages are the same in every chunk
    int g_off[C::NG];
    if constexpr (E::ESZ == 4) {
#pragma unroll
        for (int i = 0; i < C::NG; ++i) g_off[i] = g_piece(((i * NT + tid) % (FG / 4)) * 16);
    } else {
#pragma unroll
        for (int i = 0; i < C::NG / 2; ++i) g_off[i] = g_piece(((i * NT + tid) % (FG / 8)) * 16);
    }
    auto load_chunk = [&](int ci) {
        const int t0 = t_begin + ci * TC;
        if constexpr (E::ESZ == 4) {
#pragma unroll
            for (int i = 0; i < C::NG; ++i) {
                const int q = i * NT + tid;
                rg[i] = ld_g((size_t)a.N * 4, t0 + q / (FG / 4), g_off[i]);
            }
#pragma unroll
            for (int i = 0; i < C::NX; ++i) {
                const int q = i * NT + tid;
                rx[i] = ld_panel(X, (size_t)a.K * 4, x_col0, x_valid, t0 + q / (FX / 4), (q % (FX / 4)) * 16);
            }
        } else {
            // unit = (token pair, 8 features)
#pragma unroll
            for (int i = 0; i < C::NG / 2; ++i) {
                const int u = i * NT + tid;
                const int tp = u / (FG / 8), f8 = u % (FG / 8);
                (void)f8;
                rg[2 * i] = ld_g((size_t)a.N * 2, t0 + 2 * tp, g_off[i]);
                rg[2 * i + 1] = ld_g((size_t)a.N * 2, t0 + 2 * tp + 1, g_off[i]);
            }
#pragma unroll
            for (int i = 0; i < C::NX / 2; ++i) {
                const int u = i * NT + tid;
                const int tp = u / (FX / 8), f8 = u % (FX / 8);
                rx[2 * i] = ld_panel(X, (size_t)a.K * 2, x_col0, x_valid, t0 + 2 * tp, f8 * 16);
                rx[2 * i + 1] = ld_panel(X, (size_t)a.K * 2, x_col0, x_valid, t0 + 2 * tp + 1, f8 * 16);
            }
        }
    };
    auto store_chunk = [&](int buf) {
        unsigned char* sg = stage0 + buf * C::STAGE_BYTES;
        unsigned char* sx = sg + C::G_BYTES;
        if constexpr (E::ESZ == 4) {
#pragma unroll
            for (int i = 0; i < C::NG; ++i) reinterpret_cast<uint4*>(sg)[i * NT + tid] = rg[i];
#pragma unroll
            for (int i = 0; i < C::NX; ++i) reinterpret_cast<uint4*>(sx)[i * NT + tid] = rx[i];
        } else {
#pragma unroll
            for (int i = 0; i < C::NG / 2; ++i) {
                const int u = i * NT + tid;
                uint4 lo, hi;
                interleave_bf16_rows(rg[2 * i], rg[2 * i + 1], lo, hi);
                uint4* d = reinterpret_cast<uint4*>(sg) + 2 * u;   // [tp][f8*8 .. +7] words
                d[0] = lo;
                d[1] = hi;
            }
#pragma unroll
            for (int i = 0; i < C::NX / 2; ++i) {
                const int u = i * NT + tid;
                uint4 lo, hi;
                interleave_bf16_rows(rx[2 * i], rx[2 * i + 1], lo, hi);
                uint4* d = reinterpret_cast<uint4*>(sx) + 2 * u;
                d[0] = lo;
                d[1] = hi;
            }
        }
    };

    T* out = static_cast<T*>(a.out);
    float* part = a.partial ? a.partial + (size_t)sp * a.nnz * 1024 : nullptr;

    for (int q0 = 0; q0 < nq; q0 += C::QMAX) {
        // this pass: blocks [q0, q0 + npass), dealt to the waves in contiguous runs
        const int npass = (nq - q0 < C::QMAX) ? nq - q0 : C::QMAX;
        // (runs of npass / NW blocks, the first npass % NW waves one more: waves w and w + 4 share a SIMD, so the
        // longer runs spread over the SIMDs)
        const int per = npass / NW, rem = npass % NW;
        const int w_lo = q0 + wave * per + (wave < rem ? wave : rem);
        const int w_n = per + (wave < rem ? 1 : 0);

        f32x16 acc[QW];
#pragma unroll
        for (int i = 0; i < QW; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

        auto compute_chunk = [&](int buf) {
            const uint32_t* sg = reinterpret_cast<const uint32_t*>(stage0 + buf * C::STAGE_BYTES);
            const uint32_t* sx = reinterpret_cast<const uint32_t*>(stage0 + buf * C::STAGE_BYTES + C::G_BYTES);
#pragma unroll
            for (int i = 0; i < QW; ++i) {
                if (i < w_n) {
                    const int pos = __builtin_amdgcn_readfirstlane((int)s_pos[w_lo + i]);
                    const int rl = pos >> 8, cl = pos & 255;
                    const uint32_t* pa = sx + cl * 32 + lrow;   // A operand: X^T, rows = X feature j
                    const uint32_t* pb = sg + rl * 32 + lrow;   // B operand: G,   cols = G feature i
                    if constexpr (E::ESZ == 4) {
                        // 16 tokens: lane half h holds tokens 8h .. 8h+7
#pragma unroll
                        for (int s = 0; s < 8; ++s) {
                            const float av = __uint_as_float(pa[(8 * h + s) * FX]);
                            const float bv = __uint_as_float(pb[(8 * h + s) * FG]);
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i], 0, 0, 0);
                        }
                    } else {
                        // 32 tokens = 16 pair rows: lane half h holds pair rows 8h .. 8h+7
                        uint4 fa[2], fb[2];
#pragma unroll
                        for (int q = 0; q < 2; ++q) {
                            fa[q].x = pa[(8 * h + 4 * q + 0) * FX];
                            fa[q].y = pa[(8 * h + 4 * q + 1) * FX];
                            fa[q].z = pa[(8 * h + 4 * q + 2) * FX];
                            fa[q].w = pa[(8 * h + 4 * q + 3) * FX];
                            fb[q].x = pb[(8 * h + 4 * q + 0) * FG];
                            fb[q].y = pb[(8 * h + 4 * q + 1) * FG];
                            fb[q].z = pb[(8 * h + 4 * q + 2) * FG];
                            fb[q].w = pb[(8 * h + 4 * q + 3) * FG];
                        }
                        E::mma(acc[i], fa, fb);
                    }
                }
            }
        };

        if (nchunks > 0) {
            load_chunk(0);
            store_chunk(0);
            __syncthreads();
            for (int ci = 0; ci < nchunks; ++ci) {
                const bool more = ci + 1 < nchunks;
                if (more) load_chunk(ci + 1);
                compute_chunk(ci & 1);
                if (more) store_chunk((ci + 1) & 1);
                __syncthreads();
            }
        }

        // ---- store: result row j (X feature), column i (G feature) ----
#pragma unroll
        for (int i = 0; i < QW; ++i) {
            if (i < w_n) {
                const int b = __builtin_amdgcn_readfirstlane(s_blk[w_lo + i]);
                if (b >= 0) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const size_t o = (size_t)b * 1024 + acc_row(v, h) * 32 + lrow;
                        if (part) part[o] = acc[i][v];
                        else out[o] = E::from_f32(acc[i][v]);
                    }
                }
            }
        }
    }
}

// out[e] = sum over slices of partial[s][e], added in slice order.
template <typename T>
__global__ __launch_bounds__(256) void sdd_reduce_kernel(const float* partial, T* out, size_t n, int nsplit) {
    using E = Elem<T>;
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= n) return;   // n is a multiple of 1024
    // non-temporal loads: the partial sums are not read again
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    f32x4 s = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partial + i4));
    for (int k = 1; k < nsplit; ++k) s += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partial + (size_t)k * n + i4));
    out[i4 + 0] = E::from_f32(s.x);
    out[i4 + 1] = E::from_f32(s.y);
    out[i4 + 2] = E::from_f32(s.z);
    out[i4 + 3] = E::from_f32(s.w);
}

}  // namespace pbs
