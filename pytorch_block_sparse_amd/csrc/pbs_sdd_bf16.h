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
// (global_load_lds_dwordx4, contiguous in global memory) into one of NS chunk buffers, so that NS - 1
// chunks of loads are in flight while one is consumed (the operands come from HBM; a single chunk in
// flight does not cover that latency).  The rows stay
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

template <int QW, int TC_, int NS_, int NW_ = 8>
struct SddBf16Cfg {
    static constexpr int SR = 16, SC = 16, NW = NW_, NT = NW * 64;
    static constexpr int TC = TC_;                           // tokens per chunk (16 or 32)
    static constexpr int NS = NS_;                           // chunk buffers: NS - 1 chunks of loads in flight
    static constexpr int ROW_BYTES = 1024;                   // one token row of a panel: 16 blocks x 32 x 2 B
    static constexpr int PANEL_BYTES = TC * ROW_BYTES;
    static constexpr int STAGE_BYTES = 2 * PANEL_BYTES;      // G panel, then X panel
    static constexpr int LIST_MAX = SR * SC;
    static constexpr int QMAX = QW * NW;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + LIST_MAX * 4 + LIST_MAX * 2 + (2 * SR + SC / 2 + 4) * 4;
    static constexpr int ROWS_PER_WAVE = TC / NW;            // token rows of each panel a wave copies per chunk
    static_assert(TC_ == 16 || TC_ == 32, "one or two 16-token matrix steps per chunk");
    static_assert(NS_ >= 2 && NS_ <= 4, "chunk buffers");
    static_assert(QW >= ROWS_PER_WAVE, "a wave issues its token rows between its block products");
};

// The rectangle's rows, columns and block list, built by all threads of the workgroup (NT threads, of
// which the first 8 waves place the blocks).  smem: scratch of at least SDD_BF16_PROLOGUE_BYTES at the start
// of the (not yet used) chunk buffers.  Results in LDS: s_blk / s_pos (data block and (row place << 8 |
// column place) of each block, row-major), s_rowoff[SR] = number of blocks, s_rowid[SR] = block row of
// W in each row place or -1, s_gu[SC / 2] = column unit (pair of block columns) in each place or -1.
constexpr int SDD_BF16_EMAX = 8192, SDD_BF16_UMAX = 1024;
constexpr int SDD_BF16_PROLOGUE_BYTES = (2 * 16 + 1 + 2 * SDD_BF16_EMAX + 2 * SDD_BF16_UMAX + 2 * SDD_BALANCE_MAX_ROWS + 3) * 4;
template <int NT>
static __device__ __forceinline__ void sdd_bf16_prologue(const SddArgs& a, int tile, unsigned char* smem, int* s_blk,
                                                         unsigned short* s_pos, int* s_rowoff, int* s_rowid, int* s_gu) {
    constexpr int SR = 16, SC = 16, NW = 8;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c0 = (tile % a.tiles_c) * SC;
    const int nblk_r = a.N / 32;
    // ---- which rows and columns of W this rectangle covers, and the list of its blocks (row-major) ----
    // Rows: the band's 16 block rows (sdd_band_rows).  Columns: normally the band's columns c0 .. c0+15.
    // When the band's entries fit in LDS the columns of the band are instead dealt to the band's
    // rectangles by block count, in units of two adjacent columns (one 128-byte piece of an X row):
    // the units are ranked by their number of blocks in this band and handed out in serpentine order.
    // Rectangles of one band then hold the same number of blocks to within a few, instead of
    // 64 +- 7 at density 0.25, and the kernel no longer waits for its fullest rectangle.
    const int band = tile / a.tiles_c, grp = tile % a.tiles_c;
    const int nblk_c = a.K / 32;
    const int nunits = (nblk_c + 1) / 2;
    // scratch in the (not yet used) chunk buffers
    constexpr int EMAX = SDD_BF16_EMAX, UMAX = SDD_BF16_UMAX;
    int* s_lo = reinterpret_cast<int*>(smem);   // [SR] first entry of each row
    int* s_rs = s_lo + SR;                      // [SR + 1] start of each row's entries in the cached arrays
    int* s_ecol = s_rs + SR + 1;                // [EMAX] block column of each cached entry
    int* s_eblk = s_ecol + EMAX;                // [EMAX] data block of each cached entry
    int* s_cnt = s_eblk + EMAX;                 // [UMAX] blocks of the band per column unit
    int* s_ug = s_cnt + UMAX;                   // [UMAX] rectangle * 8 + place of each column unit
    int* s_scan = s_ug + UMAX;                  // [SDD_BALANCE_MAX_ROWS + 2] scratch of the row scan
    int* s_ptr_copy = s_scan + SDD_BALANCE_MAX_ROWS + 2;   // [SDD_BALANCE_MAX_ROWS + 1] row pointers, if scanned
    const bool have_ptr = sdd_band_rows(a.ptr, a.nnz, nblk_r, a.tiles_r, band, SR, s_rowid, s_scan, tid, NT, s_ptr_copy);
    __syncthreads();
    if (tid < SR) {
        const int r = s_rowid[tid];
        int lo = 0, hi = 0;
        if (r >= 0) {
            if (have_ptr) {
                lo = s_ptr_copy[r];
                hi = s_ptr_copy[r + 1];
            } else {
                lo = clamp_entry(a.ptr[r], a.nnz);
                hi = clamp_entry(a.ptr[r + 1], a.nnz);
            }
        }
        s_lo[tid] = lo;
        s_rs[tid + 1] = hi > lo ? hi - lo : 0;
    }
    if (tid < SC / 2) s_gu[tid] = -1;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        s_rs[0] = 0;
        for (int i = 0; i < SR; ++i) {
            run += s_rs[i + 1];
            s_rs[i + 1] = run;
        }
    }
    __syncthreads();
    const int nent = s_rs[SR];
    const bool cached = nent <= EMAX;
    const bool dealt = cached && nunits <= UMAX && a.tiles_c >= 2;
    int my_lo = 0, my_n = 0;
    if (cached) {
        // one sweep over the band's entries (entry i belongs to the row r with s_rs[r] <= i < s_rs[r + 1]):
        // all loads of a thread are in flight together
        for (int i = tid; i < nent; i += NT) {
            int r = 0;
#pragma unroll
            for (int k = 1; k < SR; ++k) r += (i >= s_rs[k]) ? 1 : 0;
            const int2 e = *reinterpret_cast<const int2*>(a.idx + 2 * (size_t)(s_lo[r] + i - s_rs[r]));
            s_ecol[i] = e.x;
            s_eblk[i] = e.y;
        }
        if (dealt)
            for (int u = tid; u < nunits; u += NT) s_cnt[u] = 0;
        __syncthreads();
        if (dealt) {
            for (int i = tid; i < nent; i += NT) {
                const int c = s_ecol[i];
                if (c >= 0 && c < nblk_c) atomicAdd(&s_cnt[c >> 1], 1);
            }
            __syncthreads();
            for (int u = tid; u < nunits; u += NT) {
                const int n = s_cnt[u];
                int rank = 0;
                for (int o = 0; o < nunits; ++o) {
                    const int m = s_cnt[o];
                    rank += (m > n || (m == n && o < u)) ? 1 : 0;
                }
                const int place = rank / a.tiles_c;   // < SC / 2: there are at most 8 units per rectangle
                int gsel = rank % a.tiles_c;
                if (place & 1) gsel = a.tiles_c - 1 - gsel;
                s_ug[u] = gsel * (SC / 2) + place;
                if (gsel == grp) s_gu[place] = u;
            }
        } else if (tid < SC / 2) {
            const int u = grp * (SC / 2) + tid;
            s_gu[tid] = u < nunits ? u : -1;
        }
        __syncthreads();
        // rows 2*wave and 2*wave + 1: first count this rectangle's blocks, then (below) place them
        auto mine_of = [&](int c) -> int {   // place (0..15) of block column c in this rectangle, or -1
            if (c < 0 || c >= nblk_c) return -1;
            const int ug = dealt ? s_ug[c >> 1] : (c >> 1);
            return (ug / (SC / 2)) == grp ? (ug % (SC / 2)) * 2 + (c & 1) : -1;
        };
#pragma unroll
        for (int rr = 0; rr < SR / NW; ++rr) {
            if (wave >= NW) break;
            const int r = wave * (SR / NW) + rr;
            const int off = s_rs[r], n = s_rs[r + 1] - off;
            int cnt = 0;
            for (int b0 = 0; b0 < n; b0 += 64) {
                const bool m = (b0 + lane < n) && mine_of(s_ecol[off + b0 + lane]) >= 0;
                cnt += __popcll(__ballot(m));
            }
            if (lane == 0) s_rowoff[r] = cnt < SC ? cnt : SC;   // (repeated columns: never more than the tables hold)
        }
    } else {
        if (tid < SC / 2) {
            const int u = grp * (SC / 2) + tid;
            s_gu[tid] = u < nunits ? u : -1;
        }
        if (tid < SR) {
            const int r = s_rowid[tid];
            if (r >= 0) {
                const int lo = clamp_entry(a.ptr[r], a.nnz), hi = clamp_entry(a.ptr[r + 1], a.nnz);
                int l = lo, u = hi;
                while (l < u) {   // rows are sorted by block column: first entry with column >= c0
                    const int mid = (l + u) >> 1;
                    if (a.idx[2 * mid] < c0) l = mid + 1; else u = mid;
                }
                my_lo = l;
                while (l < hi && a.idx[2 * l] < c0 + SC) ++l;
                my_n = l - my_lo;
                if (my_n > SC) my_n = SC;
            }
            s_rowoff[tid] = my_n;
        }
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
    if (cached) {
        auto mine_of = [&](int c) -> int {
            if (c < 0 || c >= nblk_c) return -1;
            const int ug = dealt ? s_ug[c >> 1] : (c >> 1);
            return (ug / (SC / 2)) == grp ? (ug % (SC / 2)) * 2 + (c & 1) : -1;
        };
#pragma unroll
        for (int rr = 0; rr < SR / NW; ++rr) {
            if (wave >= NW) break;
            const int r = wave * (SR / NW) + rr;
            const int off = s_rs[r], n = s_rs[r + 1] - off;
            int run = s_rowoff[r];
            for (int b0 = 0; b0 < n; b0 += 64) {
                const int cl = (b0 + lane < n) ? mine_of(s_ecol[off + b0 + lane]) : -1;
                const unsigned long long bal = __ballot(cl >= 0);
                const int at = run + __popcll(bal & ((1ull << lane) - 1ull));
                if (cl >= 0 && at < s_rowoff[r + 1]) {
                    int b = s_eblk[off + b0 + lane];
                    if (b < 0 || b >= a.nnz) b = -1;
                    s_blk[at] = b;
                    s_pos[at] = (unsigned short)((r << 8) | cl);
                }
                run += __popcll(bal);
            }
        }
    } else if (tid < SR) {
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
}

template <int QW, int TC_, int NS_, int NW_ = 8>
__global__ __launch_bounds__(NW_ * 64) void sdd_bf16_kernel(SddArgs a) {
    using C = SddBf16Cfg<QW, TC_, NS_, NW_>;
    constexpr int NS = C::NS;
    constexpr int SR = C::SR, SC = C::SC, NW = C::NW, TC = C::TC;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    int* s_blk = reinterpret_cast<int*>(smem + NS * C::STAGE_BYTES);                  // [LIST_MAX] data block
    unsigned short* s_pos = reinterpret_cast<unsigned short*>(s_blk + C::LIST_MAX);  // [LIST_MAX] (rl << 8) | cl
    int* s_rowoff = reinterpret_cast<int*>(s_pos + C::LIST_MAX);                     // [SR + 1]
    const unsigned lds0 = (unsigned)(uintptr_t)smem;

    const int ntiles = a.tiles_r * a.tiles_c;
    const int wg = xcd_tile_id(blockIdx.x, ntiles * a.nsplit);
    if (wg < 0) return;
    const int sp = wg / ntiles;
    const int tile = wg % ntiles;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane & 31;
    const int h = lane >> 5;

    // ---- which rows and columns of W this rectangle covers, and the list of its blocks (row-major) ----
    int* s_rowid = s_rowoff + SR + 2;   // [SR] block row of W in each place of this rectangle's band, or -1
    int* s_gu = s_rowid + SR;           // [SC / 2] column unit in each place of this rectangle, or -1
    static_assert(SDD_BF16_PROLOGUE_BYTES <= NS * C::STAGE_BYTES, "scratch fits in the chunk buffers");
    const int nblk_c = a.K / 32;
    sdd_bf16_prologue<C::NT>(a, tile, smem, s_blk, s_pos, s_rowoff, s_rowid, s_gu);
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
    const int pc = lane ^ ((wave & 3) << 2);   // panel chunk fetched by this lane
    // G: the 64 bytes of place pc / 4 of the band come from that place's block row (a place without a
    // row fetches any valid address; nothing reads it)
    const int g_rid = s_rowid[pc >> 2];
    const unsigned g_voff = g_rid >= 0 ? (unsigned)(g_rid * 64 + (pc & 3) * 16) : 0u;
    // X: the 64 bytes of place pc / 4 come from that place's block column (two adjacent columns per unit)
    const int x_unit = s_gu[pc >> 3];
    const int x_cid = x_unit >= 0 ? x_unit * 2 + ((pc >> 2) & 1) : -1;
    const unsigned x_voff = (x_cid >= 0 && x_cid < nblk_c) ? (unsigned)(x_cid * 64 + (pc & 3) * 16) : 0u;
    const size_t g_row_bytes = (size_t)a.N * 2, x_row_bytes = (size_t)a.K * 2;

    // DMA issue state: chunks are issued in order; the addresses of the chunk being issued are kept and
    // advanced by constant strides (a 64-bit multiply per row and panel cost more scalar instructions per
    // chunk than all the rest of the chunk's bookkeeping).
    const size_t g_kstep = (size_t)NW * g_row_bytes, x_kstep = (size_t)NW * x_row_bytes;   // between this wave's rows
    const size_t g_cstep = (size_t)TC * g_row_bytes, x_cstep = (size_t)TC * x_row_bytes;   // between chunks
    int iss_t = 0;                       // token of this wave's first row in the chunk being issued
    unsigned iss_stage = 0;              // LDS address of that row in the chunk's buffer
    const unsigned char* iss_g = G;      // global address of that row, G panel
    const unsigned char* iss_x = X;
    auto issue_reset = [&]() {
        iss_t = t_begin + wave;
        iss_stage = lds0 + wave * C::ROW_BYTES;
        iss_g = uniform_ptr(G + (size_t)iss_t * g_row_bytes);
        iss_x = uniform_ptr(X + (size_t)iss_t * x_row_bytes);
    };
    // token row number k of this wave's ROWS_PER_WAVE, both panels, of the chunk being issued; returns the DMA count
    auto issue_row = [&](int k) -> int {
        const int t = iss_t + k * NW;
        const unsigned stage = iss_stage + k * NW * C::ROW_BYTES;
        if (t < t_end) {
            dma16(stage, iss_g + k * g_kstep, g_voff);
            dma16(stage + C::PANEL_BYTES, iss_x + k * x_kstep, x_voff);
            return 2;
        }
        // tokens past the end contribute nothing
        unsigned char* p = smem + (stage - lds0) + lane * 16;
        *reinterpret_cast<uint4*>(p) = make_uint4(0, 0, 0, 0);
        *reinterpret_cast<uint4*>(p + C::PANEL_BYTES) = make_uint4(0, 0, 0, 0);
        return 0;
    };
    auto issue_next = [&]() {   // the next chunk goes to the next buffer
        iss_t += TC;
        iss_g += g_cstep;
        iss_x += x_cstep;
        iss_stage += C::STAGE_BYTES;
        if (iss_stage >= lds0 + NS * C::STAGE_BYTES) iss_stage -= NS * C::STAGE_BYTES;
    };
    auto issue_chunk = [&]() -> int {
        int n = 0;
#pragma unroll
        for (int k = 0; k < C::ROWS_PER_WAVE; ++k) n += issue_row(k);
        issue_next();
        return n;
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
        // (runs of npass / NW blocks, the first npass % NW waves one more: with runs of ceil(npass / NW) the last
        // wave of 66 blocks had 3 and the others 9)
        const int per = npass / NW, rem = npass % NW;
        const int w_lo = q0 + wave * per + (wave < rem ? wave : rem);
        const int w_n = per + (wave < rem ? 1 : 0);

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

        constexpr int NU = TC / 16;   // 16-token matrix steps per chunk
        auto load_frag = [&](uint4 (&f)[NU], const unsigned char* p) {
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const uint2 lo = tr16_b64(p + (16 * u) * C::ROW_BYTES);
                const uint2 hi = tr16_b64(p + (16 * u + 4) * C::ROW_BYTES);
                f[u] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        };
        // products of chunk ci, and this wave's share of the DMA of the next chunk to issue (if do_issue): in the lower
        // four waves one token row of both panels after each of the first blocks, so that the texture path works
        // while the matrix cores do (issued in one go ahead of the products, the copy instructions hold a wave for as
        // long as the texture path needs for them, and its products only start after that: what the upper four waves do
        // on purpose, see below).  Returns the number of DMA instructions issued.
        auto compute_chunk = [&](int ci, bool do_issue) -> int {
            const unsigned char* stage = smem + (ci % NS) * C::STAGE_BYTES;
            int n_dma = 0;
            // The fragments of block q + 1 are fetched before the products of block q are issued, so that the
            // LDS round trip of one block runs under the matrix instructions of the one before it (fetched
            // right before their own products, the eight or so round trips of a chunk added up to twice the
            // matrix time).  The loop is unrolled: the two fragment sets alternate by name, not by copying.
            uint4 fa[2][NU], fb[2][NU];
            if (w_n > 0) {
                load_frag(fb[0], stage + b_off[0]);
                load_frag(fa[0], stage + a_off[0]);
            }
            // The two waves of a SIMD copy at different times: the upper four waves issue their token rows in one go
            // ahead of their products (and are held by the texture path meanwhile), the lower four between their
            // first products, so that a SIMD has one wave computing while the other is held (all eight issuing
            // between their products stalled in step: 0.246 -> 0.238 ms).
            const bool early = wave >= NW / 2;
            if (early && do_issue) {
#pragma unroll
                for (int k = 0; k < C::ROWS_PER_WAVE; ++k) n_dma += issue_row(k);
            }
            const bool do_issue_between = do_issue && !early;
#pragma unroll
            for (int q = 0; q < QW; ++q) {
                if (q >= w_n && q < C::ROWS_PER_WAVE && do_issue_between) n_dma += issue_row(q);   // fewer blocks than rows to copy
                if (q < w_n) {
                    constexpr int cur = 0, nxt = 1;
                    uint4(&fa_c)[NU] = fa[(q & 1) ? nxt : cur];
                    uint4(&fb_c)[NU] = fb[(q & 1) ? nxt : cur];
                    uint4(&fa_n)[NU] = fa[(q & 1) ? cur : nxt];
                    uint4(&fb_n)[NU] = fb[(q & 1) ? cur : nxt];
                    if (q + 1 < QW && q + 1 < w_n) {
                        load_frag(fa_n, stage + a_off[q + 1]);
                        if (rl_of[q + 1] != rl_of[q]) {
                            load_frag(fb_n, stage + b_off[q + 1]);
                        } else {
#pragma unroll
                            for (int u = 0; u < NU; ++u) fb_n[u] = fb_c[u];
                        }
                    }
#pragma unroll
                    for (int u = 0; u < NU; ++u)
                        acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa_c[u]),
                                                                         __builtin_bit_cast(bf16x8, fb_c[u]), acc[q], 0, 0, 0);
                    if (q < C::ROWS_PER_WAVE && do_issue_between) n_dma += issue_row(q);
                }
            }
            if (do_issue) issue_next();
            return n_dma;
        };

        if (nchunks > 0) {
            // DMA counts of the chunks in flight, oldest (the one computed next) first
            int pend[NS];
#pragma unroll
            for (int k = 0; k < NS; ++k) pend[k] = 0;
            issue_reset();
#pragma unroll
            for (int k = 0; k < NS - 1; ++k)
                if (k < nchunks) pend[k] = issue_chunk();
            for (int ci = 0; ci < nchunks; ++ci) {
                // chunk ci has landed for every wave, and every wave is done reading chunk ci - 1
                if constexpr (NS == 2) {
                    drain_barrier();   // with two buffers nothing younger than chunk ci is in flight
                } else {
                    int later = 0;
#pragma unroll
                    for (int k = 1; k < NS; ++k) later += pend[k];
                    wait_dma_and_barrier(later);
                }
#pragma unroll
                for (int k = 0; k + 1 < NS; ++k) pend[k] = pend[k + 1];
                pend[NS - 1] = 0;
                // chunk ci + NS - 1 goes into the buffer of chunk ci - 1, which every wave has left
                pend[NS - 2] = compute_chunk(ci, ci + NS - 1 < nchunks);
            }
            lds_barrier();   // the next pass refills the buffers
        }

        // ---- store: result row j (X feature), column i (G feature) ----
#pragma unroll
        for (int q = 0; q < QW; ++q) {
            if (q < w_n && blk_of[q] >= 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const size_t o = (size_t)blk_of[q] * 1024 + acc_row(v, h) * 32 + lrow;
                    // (partial sums are written once and read once, by sdd_reduce_kernel: stored and loaded non-temporally
                    // they leave the operands of the next product in the last-level cache)
                    if (part) __builtin_nontemporal_store(acc[q][v], part + o);
                    else out[o] = Elem<bf16_t>::from_f32(acc[q][v]);
                }
            }
        }
    }
}

}  // namespace pbs
