// dense^T x dense -> block-sparse, fp32, with the blocks of a row band cut into equal shares.
//
// The rectangle kernel (pbs_sdd.h) gives a workgroup whatever blocks its rectangle of positions
// happens to hold.  Its time per chunk of tokens is set by its busiest wave, ceil(blocks / 8) products
// of 1024 matrix-core cycles, and the launch ends with its fullest rectangle: at density 0.25 a
// 16 x 8 rectangle holds 32 +- 5 blocks, the fullest of 128 about 47, i.e. 6 rounds for 4 rounds of
// mean work.  Here a band of up to SR block rows is cut into `segs` segments of the SAME number of
// blocks (+- 1): the band's blocks are ranked column-major (by block column, then by row within the
// band), and segment j takes ranks [N j / segs, N (j + 1) / segs).  A segment covers a run of whole
// columns plus a part of the first and of the last one; its X panel starts at its first column.  The
// host picks `segs` so that a segment's share is at most 8 x rounds for a whole number of rounds
// (plan_sdd_seg), and every workgroup of the launch then does the same number of rounds.
//
// Every workgroup of a band derives the same cut from the band's CSR entries: a histogram of the
// block columns in LDS, its prefix sum, and for the two boundary columns the rows that hold them.
// A segment whose columns exceed the panel's SC columns (sparser stretches of the pattern) is done in
// several windows of SC columns, each streaming the tokens again: correct, slower, rare.
#pragma once
#include "pbs_common.h"
#include "pbs_sdd.h"
#include <type_traits>

namespace pbs {

template <int SR, int SC, int QW, int NW>
struct SddSegCfg {
    static constexpr int NT = NW * 64;
    static constexpr int TC = 16;                           // tokens per staged chunk
    static constexpr int FG = SR * 32;                      // features per token row, G panel
    static constexpr int FX = SC * 32;
    static constexpr int G_BYTES = TC * FG * 4;
    static constexpr int X_BYTES = TC * FX * 4;
    static constexpr int STAGE_BYTES = G_BYTES + X_BYTES;
    static constexpr int QMAX = QW * NW;
    static constexpr int LIST_MAX = SR * SC;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES + (LIST_MAX + SR + 4) * 4;
    static constexpr int MAX_COLS = 2 * STAGE_BYTES / 4 - 64;   // the column histogram borrows the stage buffers
    static_assert(SR <= 64 && SC <= 255, "list entry packs (row place, column) in bytes");
    static constexpr int G_DMA = G_BYTES / 1024 / NW;     // DMA instructions (1 KB each) per wave and chunk
    static constexpr int X_DMA = X_BYTES / 1024 / NW;
    static_assert(G_BYTES % (1024 * NW) == 0 && X_BYTES % (1024 * NW) == 0, "the waves copy equal shares of both panels");
};

template <int SR, int SC, int QW, int NW>
__global__ __launch_bounds__(NW * 64) void sdd_seg_kernel(SddArgs a) {
    using C = SddSegCfg<SR, SC, QW, NW>;
    using E = Elem<float>;
    constexpr int NT = C::NT, TC = C::TC, FG = C::FG, FX = C::FX;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* stage0 = smem;
    int* s_blk = reinterpret_cast<int*>(smem + 2 * C::STAGE_BYTES);   // [LIST_MAX] data block id
    __shared__ unsigned short s_pos[C::LIST_MAX];                     // (row place << 8) | column - window start
    int* s_rowoff = s_blk + C::LIST_MAX;                              // [SR + 1]
    __shared__ int s_count;
    __shared__ int s_rowid[SR];      // block row of W in each place of this band, or -1
    __shared__ int s_lo[SR], s_hi[SR];
    __shared__ int s_has[2][SR];     // whether the row holds the segment's first / last column
    __shared__ int s_seg[4];         // first column, last column, ranks to skip in the first, ranks to take of the last

    const int ntiles = a.tiles_r * a.segs;
    const int wg = xcd_tile_id(blockIdx.x, ntiles * a.nsplit);
    if (wg < 0) return;
    const int sp = wg / ntiles;            // token slice: slices of one segment land on different XCDs
    const int tile = wg % ntiles;
    const int band = tile / a.segs;
    const int seg = tile % a.segs;
    const int nblk_r = a.N / 32, ncols = a.K / 32;
    const int rows_per_band = (nblk_r + a.tiles_r - 1) / a.tiles_r;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane & 31;
    const int h = lane >> 5;

    // ---- the band's rows and their entries ----
    sdd_band_rows(a.ptr, a.nnz, nblk_r, a.tiles_r, band, SR, s_rowid, reinterpret_cast<int*>(smem), tid, NT, nullptr,
                  rows_per_band);
    if (tid < SR) {
        const int r = s_rowid[tid];
        int lo = 0, hi = 0;
        if (r >= 0) {
            lo = clamp_entry(a.ptr[r], a.nnz);
            hi = clamp_entry(a.ptr[r + 1], a.nnz);
            if (hi < lo) hi = lo;
        }
        s_lo[tid] = lo;
        s_hi[tid] = hi;
    }
    // ---- blocks per column of the band, then the exclusive prefix sum: column-major ranks ----
    int* s_cnt = reinterpret_cast<int*>(smem);   // [ncols + 1]
    __syncthreads();
    for (int i = tid; i <= ncols; i += NT) s_cnt[i] = 0;
    __syncthreads();
    for (int i = 0; i < SR; ++i) {
        const int hi = s_hi[i];
        for (int e = s_lo[i] + tid; e < hi; e += NT) {
            const int c = a.idx[2 * (size_t)e];
            if (c >= 0 && c < ncols) atomicAdd(&s_cnt[c], 1);
        }
    }
    __syncthreads();
    if (wave == 0) {
        int carry = 0;
        for (int base = 0; base < ncols; base += 64) {
            const int c = base + lane;
            const int v = c < ncols ? s_cnt[c] : 0;
            int incl = v;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int o = __shfl_up(incl, d, 64);
                if (lane >= d) incl += o;
            }
            if (c < ncols) s_cnt[c] = carry + incl - v;
            carry += __shfl(incl, 63, 64);
        }
        if (lane == 0) s_cnt[ncols] = carry;
    }
    __syncthreads();
    const int n_band = s_cnt[ncols];
    const int start = (int)((long long)n_band * seg / a.segs);
    const int end = (int)((long long)n_band * (seg + 1) / a.segs);
    if (start >= end) return;   // the same for every thread
    for (int c = tid; c < ncols; c += NT) {
        const int lo = s_cnt[c], hi = s_cnt[c + 1];
        if (lo <= start && start < hi) {
            s_seg[0] = c;
            s_seg[2] = start - lo;
        }
        if (lo <= end - 1 && end - 1 < hi) {
            s_seg[1] = c;
            s_seg[3] = end - lo;
        }
    }
    __syncthreads();
    const int c_lo = s_seg[0], c_hi = s_seg[1], skip_lo = s_seg[2], take_hi = s_seg[3];
    // entry k of the row in `place`
    auto col_of = [&](int place, int k) -> int { return a.idx[2 * (size_t)(s_lo[place] + k)]; };
    auto blk_of = [&](int place, int k) -> int { return a.idx[2 * (size_t)(s_lo[place] + k) + 1]; };
    // first entry of the row in `place` whose column is >= c (entries of a row are sorted by column)
    auto lower_bound = [&](int place, int c) -> int {
        int l = 0, u = s_hi[place] - s_lo[place];
        while (l < u) {
            const int mid = (l + u) >> 1;
            if (col_of(place, mid) < c) l = mid + 1; else u = mid;
        }
        return l;
    };
    if (tid < SR) {
        const int n = s_hi[tid] - s_lo[tid];
        const int k0 = lower_bound(tid, c_lo), k1 = lower_bound(tid, c_hi);
        s_has[0][tid] = (k0 < n && col_of(tid, k0) == c_lo) ? 1 : 0;
        s_has[1][tid] = (k1 < n && col_of(tid, k1) == c_hi) ? 1 : 0;
    }
    __syncthreads();
    const int t_begin = sp * a.tokens_per_split;
    int t_end = t_begin + a.tokens_per_split;
    if (t_end > a.M) t_end = a.M;
    const int nchunks = t_begin < t_end ? (t_end - t_begin + TC - 1) / TC : 0;

    const unsigned char* G = static_cast<const unsigned char*>(a.g);
    const unsigned char* X = static_cast<const unsigned char*>(a.x);
    float* out = static_cast<float*>(a.out);
    float* part = a.partial ? a.partial + (size_t)sp * a.nnz * 1024 : nullptr;

    for (int cw = c_lo; cw <= c_hi; cw += SC) {   // windows of SC columns; almost always one
        // ---- list this segment's blocks inside the window, row-major ----
        int rank_lo = 0, rank_hi = 0;   // this row's rank within the segment's first / last column
        if (tid < SR) {
            for (int i = 0; i < tid; ++i) {
                rank_lo += s_has[0][i];
                rank_hi += s_has[1][i];
            }
        }
        auto in_segment = [&](int c) -> bool {
            bool inc = c >= c_lo && c <= c_hi;
            if (c == c_lo) inc = inc && rank_lo >= skip_lo;
            if (c == c_hi) inc = inc && rank_hi < take_hi;
            return inc;
        };
        int my_lo = 0, my_n = 0;
        const int my_len = tid < SR ? s_hi[tid] - s_lo[tid] : 0;
        if (tid < SR && s_rowid[tid] >= 0) {
            my_lo = lower_bound(tid, cw);
            for (int k = my_lo; k < my_len; ++k) {
                const int c = col_of(tid, k);
                if (c >= cw + SC || c > c_hi) break;
                my_n += in_segment(c) ? 1 : 0;
            }
            if (my_n > SC) my_n = SC;   // (a list with repeated columns: never more entries than the tables hold)
        }
        if (tid < SR) s_rowoff[tid] = my_n;
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
        if (tid < SR && my_n > 0) {
            int o = s_rowoff[tid];
            for (int k = my_lo; k < my_len; ++k) {
                const int c = col_of(tid, k);
                if (c >= cw + SC || c > c_hi) break;
                if (!in_segment(c)) continue;
                if (o >= s_rowoff[tid] + my_n) break;
                int b = blk_of(tid, k);
                if (b < 0 || b >= a.nnz) b = -1;
                s_blk[o] = b;
                s_pos[o] = (unsigned short)((tid << 8) | (c - cw));
                ++o;
            }
        }
        __syncthreads();
        const int nq = s_count;
        if (nq == 0) continue;   // the same for every thread

        const size_t x_col0 = (size_t)cw * 128;
        const int x_valid = (a.K - cw * 32) * 4;   // bytes of an X row from the window's first column to the matrix edge
        // Chunks go global -> LDS by DMA, no registers in between: every wave fetches an eighth of both panels,
        // 1 KB per instruction (lane l: 16 bytes; the token row and the feature follow from the byte's place in
        // the panel).  Places of the band that hold no row and columns past the matrix edge fetch some valid
        // address instead: no listed block reads them.  Token rows past the end of the slice (a ragged last chunk) fetch the last valid row and are then
        // overwritten with zeros in LDS before the products.
        const unsigned lds_stage = (unsigned)(uintptr_t)stage0;
        auto dma_chunk = [&](int ci, int buf) __attribute__((always_inline)) {
            const int t0 = t_begin + ci * TC;
            const int t_last = t_end - 1 - t0;   // last token row of the chunk that exists (>= 0)
            const unsigned char* src_g = uniform_ptr(G + (size_t)t0 * a.N * 4);
            const unsigned char* src_x = uniform_ptr(X + (size_t)t0 * a.K * 4 + x_col0);
            const unsigned lg = lds_stage + buf * C::STAGE_BYTES;
            const unsigned lx = lg + C::G_BYTES;
            // the panels are linear in LDS ([token][feature]); instruction j fills bytes 1024 j .. + 1024
#pragma unroll
            for (int k = 0; k < C::G_DMA; ++k) {
                const int j = wave * C::G_DMA + k;
                const int pb = j * 1024 + lane * 16;
                int t = pb / (FG * 4);
                const int off = pb % (FG * 4);
                t = t < t_last ? t : t_last;
                const int rid = s_rowid[off / 128];
                dma16(lg + j * 1024, src_g, (unsigned)(t * a.N * 4 + (rid < 0 ? 0 : rid) * 128 + off % 128));
            }
#pragma unroll
            for (int k = 0; k < C::X_DMA; ++k) {
                const int j = wave * C::X_DMA + k;
                const int pb = j * 1024 + lane * 16;
                int t = pb / (FX * 4);
                const int off = pb % (FX * 4);
                t = t < t_last ? t : t_last;
                dma16(lx + j * 1024, src_x, (unsigned)(t * a.K * 4 + (off < x_valid ? off : 0)));
            }
        };
        // zero the token rows of chunk ci that lie past the end of the slice (all threads; barrier included)
        auto zero_tail = [&](int ci, int buf) {
            const int valid = t_end - (t_begin + ci * TC);   // token rows of the chunk that exist
            if (valid >= TC) return;                          // the same for every thread
            uint4* sg = reinterpret_cast<uint4*>(stage0 + buf * C::STAGE_BYTES);
            uint4* sx = reinterpret_cast<uint4*>(stage0 + buf * C::STAGE_BYTES + C::G_BYTES);
            for (int i = valid * (FG / 4) + tid; i < TC * (FG / 4); i += NT) sg[i] = make_uint4(0, 0, 0, 0);
            for (int i = valid * (FX / 4) + tid; i < TC * (FX / 4); i += NT) sx[i] = make_uint4(0, 0, 0, 0);
            __syncthreads();
        };

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

            // where this wave's blocks sit in the panels (the same in every chunk): scalar registers
            int pos[QW];
#pragma unroll
            for (int i = 0; i < QW; ++i) pos[i] = i < w_n ? __builtin_amdgcn_readfirstlane((int)s_pos[w_lo + i]) : 0;

            // The 16 fragment values of a block's 8 products (16 tokens: lane half h holds tokens 8h .. 8h+7) are
            // fetched together, one block ahead of the products that use them, so a wave pays one LDS round trip
            // per 512 matrix-core cycles and that one behind the previous block's products.  The blocks are
            // nested (block i + 1 is only ever reached from block i), so each path is straight-line code and the
            // waits can count exactly.
            auto fetch_frags = [&](const uint32_t* sg, const uint32_t* sx, int p, float (&av)[8], float (&bv)[8]) __attribute__((always_inline)) {
                const int rl = p >> 8, cl = p & 255;
                const uint32_t* pa = sx + cl * 32 + lrow + 8 * h * FX;   // A operand: X^T, rows = X feature j
                const uint32_t* pb = sg + rl * 32 + lrow + 8 * h * FG;   // B operand: G,   cols = G feature i
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    av[s] = __uint_as_float(pa[s * FX]);
                    bv[s] = __uint_as_float(pb[s * FG]);
                }
            };
            // next_ci >= 0: this wave's share of the DMA of that chunk is issued behind the first (upper four waves:
            // second) block's products, so that the matrix cores are already busy while the wave spends its issue
            // slots on the DMA
            auto compute_chunk = [&](int buf, int next_ci) __attribute__((always_inline)) {
                const uint32_t* sg = reinterpret_cast<const uint32_t*>(stage0 + buf * C::STAGE_BYTES);
                const uint32_t* sx = reinterpret_cast<const uint32_t*>(stage0 + buf * C::STAGE_BYTES + C::G_BYTES);
                float av[2][8], bv[2][8];
                // block I: fetch block I + 1's fragments (the last block fetches its own again: no branch around
                // the loads), then the 8 products of block I; the scheduling barriers keep that order
#define PBS_SEG_BLOCK(I)                                                                                              \
    if constexpr ((I) < QW) {                                                                                         \
        if ((I) < w_n) {                                                                                              \
            if constexpr ((I) + 1 < QW)                                                                               \
                fetch_frags(sg, sx, (I) + 1 < w_n ? pos[((I) + 1) % QW] : pos[(I) % QW], av[((I) + 1) & 1], bv[((I) + 1) & 1]); \
            __builtin_amdgcn_sched_barrier(0);                                                                        \
            _Pragma("unroll") for (int s = 0; s < 8; ++s)                                                             \
                acc[(I) % QW] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[(I) & 1][s], bv[(I) & 1][s], acc[(I) % QW], 0, 0, 0); \
            __builtin_amdgcn_sched_barrier(0);                                                                        \
            if ((I) < 2 && (I) == dma_at && next_ci >= 0) dma_chunk(next_ci, next_ci & 1);
#define PBS_SEG_END }}

                static_assert(QW <= 10, "the nest below has ten levels");
                // the two waves of a SIMD copy at different times (the upper four waves one block later): while one is
                // held by the texture path the other has products to issue
                const int dma_at = (wave >= NW / 2 && w_n > 1) ? 1 : 0;
                if (w_n > 0) {
                    fetch_frags(sg, sx, pos[0], av[0], bv[0]);
                    PBS_SEG_BLOCK(0) PBS_SEG_BLOCK(1) PBS_SEG_BLOCK(2) PBS_SEG_BLOCK(3) PBS_SEG_BLOCK(4)
                    PBS_SEG_BLOCK(5) PBS_SEG_BLOCK(6) PBS_SEG_BLOCK(7) PBS_SEG_BLOCK(8) PBS_SEG_BLOCK(9)
                    PBS_SEG_END PBS_SEG_END PBS_SEG_END PBS_SEG_END PBS_SEG_END
                    PBS_SEG_END PBS_SEG_END PBS_SEG_END PBS_SEG_END PBS_SEG_END
                }
#undef PBS_SEG_BLOCK
#undef PBS_SEG_END
            };

            __syncthreads();   // the stage buffers may still be read (previous pass) or hold the histogram
            if (nchunks > 0) {
                dma_chunk(0, 0);
                drain_barrier();
                for (int ci = 0; ci < nchunks; ++ci) {
                    zero_tail(ci, ci & 1);
                    if (w_n == 0 && ci + 1 < nchunks) dma_chunk(ci + 1, (ci + 1) & 1);   // a wave without blocks still copies
                    compute_chunk(ci & 1, ci + 1 < nchunks ? ci + 1 : -1);
                    drain_barrier();
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
        __syncthreads();   // the lists are rebuilt for the next window
    }
}

}  // namespace pbs
