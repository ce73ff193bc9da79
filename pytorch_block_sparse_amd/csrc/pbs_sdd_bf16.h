// bf16 weight gradient on the sparse support, DMA + transposing-read version.
//
//   out[32b + j][i] = sum_t G[t][32r + i] * X[t][32c + j]   for every data block b at (r, c).
//
// One workgroup (8 waves) owns a 16 x 16 rectangle of block positions of W and one slice of the
// tokens.  The blocks present in the rectangle are listed row-major and dealt to the waves in equal
// contiguous runs (at most QW accumulators per wave; denser rectangles take further passes).
//
// Tokens are streamed in chunks of 32.  A chunk is 32 token rows of G (16 block rows = 1 KB per
// token) and of X (16 block columns = 1 KB per token): each row is one DMA instruction
// (global_load_lds_dwordx4, contiguous in global memory), double buffered.  The rows stay
// token-major in LDS; both MFMA operands need 8 consecutive tokens per lane, which
// ds_read_b64_tr_b16 gathers from 4 consecutive token rows.  One such read takes 64 bytes from each of
// 4 consecutive token rows per half wave; to put those on different banks the 16-byte chunks of token
// row t are stored at chunk position c ^ ((t & 3) << 2), i.e. shifted by multiples of 64 bytes.
//
// Consecutive blocks of a wave mostly share their block row, so the G fragment is reloaded only
// when the row changes.  Tokens past the end are zero rows written by the waves themselves.
#pragma once
#include "pbs_common.h"
#include "pbs_sdd.h"

namespace pbs {

template <int QW>
struct SddBf16Cfg {
    static constexpr int SR = 16, SC = 16, NW = 8, NT = NW * 64, TC = 32;
    static constexpr int ROW_BYTES = 1024;                   // one token row of a panel: 16 blocks x 32 x 2 B
    static constexpr int PANEL_BYTES = TC * ROW_BYTES;       // 32 KB
    static constexpr int STAGE_BYTES = 2 * PANEL_BYTES;      // G panel, then X panel
    static constexpr int LIST_MAX = SR * SC;
    static constexpr int QMAX = QW * NW;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES + LIST_MAX * 4 + LIST_MAX * 2 + (2 * SR + 4) * 4;
    static constexpr int ROWS_PER_WAVE = TC / NW;            // token rows of each panel a wave copies per chunk
};

template <int QW>
__global__ __launch_bounds__(512) void sdd_bf16_kernel(SddArgs a) {
    using C = SddBf16Cfg<QW>;
    constexpr int SR = C::SR, SC = C::SC, NW = C::NW, TC = C::TC;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    int* s_blk = reinterpret_cast<int*>(smem + 2 * C::STAGE_BYTES);                  // [LIST_MAX] data block
    unsigned short* s_pos = reinterpret_cast<unsigned short*>(s_blk + C::LIST_MAX);  // [LIST_MAX] (rl << 8) | cl
    int* s_rowoff = reinterpret_cast<int*>(s_pos + C::LIST_MAX);                     // [SR + 1]
    const unsigned lds0 = (unsigned)(uintptr_t)smem;

    const int ntiles = a.tiles_r * a.tiles_c;
    const int wg = xcd_tile_id(blockIdx.x, ntiles * a.nsplit);
    if (wg < 0) return;
    const int sp = wg / ntiles;
    const int tile = wg % ntiles;
    const int c0 = (tile % a.tiles_c) * SC;
    const int nblk_r = a.N / 32;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane & 31;
    const int h = lane >> 5;

    // ---- list the blocks of the rectangle, row-major ----
    int* s_rowid = s_rowoff + SR + 2;   // [SR] block row of W in each place of this rectangle's band, or -1
    int my_lo = 0, my_n = 0;
    sdd_band_rows(a.ptr, nblk_r, a.tiles_r, tile / a.tiles_c, SR, s_rowid, reinterpret_cast<int*>(smem), tid, C::NT);
    if (tid < SR) {
        const int r = s_rowid[tid];
        if (r >= 0) {
            const int lo = a.ptr[r], hi = a.ptr[r + 1];
            int l = lo, u = hi;
            while (l < u) {   // rows are sorted by block column: first entry with column >= c0
                const int mid = (l + u) >> 1;
                if (a.idx[2 * mid] < c0) l = mid + 1; else u = mid;
            }
            my_lo = l;
            while (l < hi && a.idx[2 * l] < c0 + SC) ++l;
            my_n = l - my_lo;
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
    const int nq = __builtin_amdgcn_readfirstlane(s_rowoff[SR]);
    if (nq == 0) return;

    const int t_begin = sp * a.tokens_per_split;
    int t_end = t_begin + a.tokens_per_split;
    if (t_end > a.M) t_end = a.M;
    const int nchunks = t_begin < t_end ? (t_end - t_begin + TC - 1) / TC : 0;

    // ---- DMA address pattern: this wave copies token rows wave, wave + 8, ... of both panels; the
    //      chunk swizzle of those rows is the same ((wave & 3) << 2) ----
    const unsigned char* G = static_cast<const unsigned char*>(a.g);
    const unsigned char* X = static_cast<const unsigned char*>(a.x);
    const int x_valid = (a.K - c0 * 32) * 2;
    const int pc = lane ^ ((wave & 3) << 2);   // panel chunk fetched by this lane
    // G: the 64 bytes of place pc / 4 of the band come from that place's block row (a place without a
    // row fetches any valid address; nothing reads it)
    const int g_rid = s_rowid[pc >> 2];
    const unsigned g_voff = g_rid >= 0 ? (unsigned)(g_rid * 64 + (pc & 3) * 16) : 0u;
    const unsigned x_voff = (pc * 16 < x_valid) ? pc * 16 : 0;
    const size_t g_row_bytes = (size_t)a.N * 2, x_row_bytes = (size_t)a.K * 2;
    const unsigned char* g_col = G;
    const unsigned char* x_col = X + (size_t)c0 * 64;

    auto issue_chunk = [&](int ci) {
        const int t0 = t_begin + ci * TC;
        const unsigned stage = lds0 + (ci & 1) * C::STAGE_BYTES;
#pragma unroll
        for (int k = 0; k < C::ROWS_PER_WAVE; ++k) {
            const int tl = wave + k * NW;
            const int t = t0 + tl;
            if (t < t_end) {
                dma16(stage + tl * C::ROW_BYTES, uniform_ptr(g_col + (size_t)t * g_row_bytes), g_voff);
                dma16(stage + C::PANEL_BYTES + tl * C::ROW_BYTES, uniform_ptr(x_col + (size_t)t * x_row_bytes), x_voff);
            } else {
                // tokens past the end contribute nothing
                unsigned char* p = smem + (ci & 1) * C::STAGE_BYTES + tl * C::ROW_BYTES + lane * 16;
                *reinterpret_cast<uint4*>(p) = make_uint4(0, 0, 0, 0);
                *reinterpret_cast<uint4*>(p + C::PANEL_BYTES) = make_uint4(0, 0, 0, 0);
            }
        }
    };

    // ---- per-lane part of the fragment addresses ----
    // transposing read: within 16 lanes, lane s addresses 4 consecutive features of token row s/4 and
    // receives, for its own feature, the 4 token rows as 4 consecutive k.  Lane l serves feature
    // (l & 31) of the block; lane half h serves tokens 8h..8h+7 of each 16-token MFMA step.
    const int l16 = lane & 15;
    const int trow = 8 * h + (l16 >> 2);                              // + 16u + 4v
    const int cb = 2 * ((lane >> 4) & 1) + ((l16 & 3) >> 1);          // 16-byte chunk inside the block's 64 bytes
    const int xr = ((l16 >> 2) & 3) << 2;                             // swizzle of token row trow (+ multiples of 4)
    const int lane_const = trow * C::ROW_BYTES + (l16 & 1) * 8;
    auto frag_off = [&](int blk16) -> int { return lane_const + (((blk16 * 4 + cb) ^ xr) * 16); };

    bf16_t* out = static_cast<bf16_t*>(a.out);
    float* part = a.partial ? a.partial + (size_t)sp * a.nnz * 1024 : nullptr;

    for (int q0 = 0; q0 < nq; q0 += C::QMAX) {
        // this pass: blocks [q0, q0 + npass), dealt to the waves in contiguous runs
        const int npass = (nq - q0 < C::QMAX) ? nq - q0 : C::QMAX;
        const int per = (npass + NW - 1) / NW;
        const int w_lo = q0 + wave * per;
        int w_n = q0 + npass - w_lo;
        if (w_n > per) w_n = per;
        if (w_n < 0) w_n = 0;

        // per accumulator slot: fragment offsets of its X block (A operand) and G block (B operand)
        int a_off[QW], b_off[QW], rl_of[QW], blk_of[QW];
#pragma unroll
        for (int q = 0; q < QW; ++q) {
            const int pos = q < w_n ? __builtin_amdgcn_readfirstlane((int)s_pos[w_lo + q]) : 0;
            rl_of[q] = pos >> 8;
            a_off[q] = C::PANEL_BYTES + frag_off(pos & 255);
            b_off[q] = frag_off(pos >> 8);
            blk_of[q] = q < w_n ? __builtin_amdgcn_readfirstlane(s_blk[w_lo + q]) : -1;
        }

        f32x16 acc[QW];
#pragma unroll
        for (int q = 0; q < QW; ++q)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[q][v] = 0.f;

        auto load_frag = [&](uint4 (&f)[2], const unsigned char* p) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const uint2 lo = tr16_b64(p + (16 * u) * C::ROW_BYTES);
                const uint2 hi = tr16_b64(p + (16 * u + 4) * C::ROW_BYTES);
                f[u] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        };
        auto compute_chunk = [&](int ci) {
            const unsigned char* stage = smem + (ci & 1) * C::STAGE_BYTES;
            uint4 fb[2];
            int cur_rl = -1;
#pragma unroll
            for (int q = 0; q < QW; ++q) {
                if (q < w_n) {
                    if (rl_of[q] != cur_rl) {
                        load_frag(fb, stage + b_off[q]);
                        cur_rl = rl_of[q];
                    }
                    uint4 fa[2];
                    load_frag(fa, stage + a_off[q]);
                    Elem<bf16_t>::mma(acc[q], fa, fb);
                }
            }
        };

        if (nchunks > 0) {
            issue_chunk(0);
            for (int ci = 0; ci < nchunks; ++ci) {
                // only chunk ci is in flight here; the other buffer was read by chunk ci-1
                drain_barrier();
                if (ci + 1 < nchunks) issue_chunk(ci + 1);
                compute_chunk(ci);
            }
            lds_barrier();   // the next pass refills buffer 0
        }

        // ---- store: result row j (X feature), column i (G feature) ----
#pragma unroll
        for (int q = 0; q < QW; ++q) {
            if (q < w_n && blk_of[q] >= 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const size_t o = (size_t)blk_of[q] * 1024 + acc_row(v, h) * 32 + lrow;
                    if (part) part[o] = acc[q][v];
                    else out[o] = Elem<bf16_t>::from_f32(acc[q][v]);
                }
            }
        }
    }
}

}  // namespace pbs
