// dense x block-sparse -> dense for bf16, wide-tile persistent version (forward and input gradient).
//
// The operand stream, not the matrix cores, bounds this product: per k-block a tile of BM tokens x NB
// block columns fetches BM x 32 dense elements plus the packed blocks present, and multiplies only
// with those.  Bytes per multiply-add fall with the number of block columns a fetched panel serves,
// so the tile is 128 tokens x 16 block columns (the accumulators of 8 waves: 2 token slices of 64 x 4
// column quarters of 4 block columns, 128 registers per lane), and the dense operand is fetched in
// 128-byte row pieces (two adjacent k-blocks, a "k-pair", per step), which the texture path moves
// about 1.5x faster than 64-byte pieces.
//
// Persistent workgroups.  A workgroup keeps one group of 16 block columns (its plan records stay in
// LDS) and walks several token tiles.  The 4 copy waves issue the DMA of the following steps across
// tile boundaries while the 8 compute waves are still in the epilogue of the previous tile, so the
// first-load latency of a tile and the store burst of its epilogue overlap with useful work.
//
// Plan (built by dds16_plan_kernel per pattern and direction): per group of 16 block columns, one
// 256-byte record per k-pair that any of them touches:
//   [0..15]  data block of each column in the even k-block of the pair, or -1
//   [16..31] the same for the odd k-block
//   [32] k-pair index   [33] presence mask (bit 16*odd + column)   [34] entries before this pair
// preceded by a header record ([0] = pairs present, [1] = entries) and followed by a sentinel
// ([34] = entries).  Entries are numbered in mask-bit order; entry e lives in block slot e % RB.
//
// LDS: [A ring: RS steps x 16 KB][block ring: RB x 2 KB][epilogue staging: 8 x 2304 B][plan records].
// Panel rows are 128 bytes (8 chunks of 16 bytes); chunk c of row r sits at position c ^ ((r >> 1) & 7),
// which makes the 16-byte fragment reads of 16 consecutive rows conflict-free.  Packed blocks are laid
// out as in the narrow kernel (pbs_dds.h).
#pragma once
#include "pbs_common.h"
#include "pbs_dds.h"

namespace pbs {

constexpr int D16_NB = 16;      // block columns per tile
constexpr int D16_REC = 64;     // ints per plan record
constexpr int D16_F_PAIR = 32, D16_F_MASK = 33, D16_F_CUM = 34;
constexpr int D16_BM = 128;     // tokens per tile
static inline size_t dds16_plan_group_ints(int KB) { return ((size_t)(KB / 2) + 2) * D16_REC; }

// One workgroup per group of 16 block columns merges their sorted block lists into k-pair records.
__global__ __launch_bounds__(256) void dds16_plan_kernel(const int32_t* __restrict__ ptr, const int32_t* __restrict__ idx,
                                                         int nblk_n, int KB, int nnz, int* plan, int group_ints) {
    constexpr int NB = D16_NB, SEG = 128, NT = 256, R = D16_REC;
    __shared__ int s_tbl[SEG * NB];
    __shared__ int s_ptr[NB + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nb0 = blockIdx.x * NB;
    int* out = plan + (size_t)blockIdx.x * group_ints;
    int* rec = out + R;
    if (tid <= NB) {
        const int nb = nb0 + tid;
        s_ptr[tid] = ptr[nb < nblk_n ? nb : nblk_n];
    }
    __syncthreads();
    const int e_begin = s_ptr[0], e_end = s_ptr[NB];
    int np = 0, ne = 0;   // running totals (kept by every thread of wave 0)
    for (int seg0 = 0; seg0 < KB; seg0 += SEG) {
        for (int i = tid; i < SEG * NB; i += NT) s_tbl[i] = -1;
        __syncthreads();
        for (int e = e_begin + tid; e < e_end; e += NT) {
            const int kb = idx[2 * e] - seg0;
            const int b = idx[2 * e + 1];
            if (kb >= 0 && kb < SEG && kb + seg0 < KB && b >= 0 && b < nnz) {
                int nl = 0;
#pragma unroll
                for (int i = 1; i < NB; ++i) nl += (e >= s_ptr[i]) ? 1 : 0;
                s_tbl[kb * NB + nl] = b;
            }
        }
        __syncthreads();
        if (wave == 0) {
            // lane = k-pair of this segment
            unsigned present = 0;
#pragma unroll
            for (int j = 0; j < 2 * NB; ++j) present |= (s_tbl[lane * 2 * NB + j] >= 0) ? (1u << j) : 0u;
            const int cnt = __popc(present);
            const unsigned long long m = __ballot(cnt != 0);
            int incl = cnt;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int o = __shfl_up(incl, d, 64);
                if (lane >= d) incl += o;
            }
            const int total = __shfl(incl, 63, 64);
            if (cnt) {
                int* r = rec + (size_t)(np + __popcll(m & ((1ull << lane) - 1ull))) * R;
#pragma unroll
                for (int j = 0; j < 2 * NB; ++j) r[j] = s_tbl[lane * 2 * NB + j];
                r[D16_F_PAIR] = seg0 / 2 + lane;
                r[D16_F_MASK] = (int)present;
                r[D16_F_CUM] = ne + incl - cnt;
#pragma unroll
                for (int j = D16_F_CUM + 1; j < R; ++j) r[j] = 0;
            }
            np += __popcll(m);
            ne += total;
        }
        __syncthreads();
    }
    if (wave == 0) {
        out[lane] = lane == 0 ? np : (lane == 1 ? ne : 0);
        int* r = rec + (size_t)np * R;   // sentinel
        r[lane] = lane < 2 * NB ? -1 : (lane == D16_F_CUM ? ne : 0);
    }
}

struct D16Args {
    const void* a;         // [M, K] row-major bf16
    const void* data;      // [nnz*32, 32] bf16
    const int* plan;       // built by dds16_plan_kernel for this pattern and direction
    const void* bias;      // nullptr or [N]
    void* out;             // [M, N] row-major
    int M, N, K, nnz;
    int m_tiles, n_groups, group_ints;
    int wg_per_group;      // workgroups that share the token tiles of one column group
};

template <int RS, int RB, int NP>
struct D16Cfg {
    static constexpr int NW = 8, NT = (NW + NP) * 64, BM = D16_BM, TM = 2, NBW = 4;
    static constexpr int ROWB = 128;                          // one panel row: 64 k values
    static constexpr int PANEL_BYTES = BM * ROWB;             // 16 KB per step
    static constexpr int A_PER_WAVE = PANEL_BYTES / 1024 / NP;
    static constexpr int COLS_PER_COPIER = D16_NB / NP;
    static constexpr int BLK_BYTES = 2048;
    static constexpr int A_RING_BYTES = RS * PANEL_BYTES;
    static constexpr int B_RING_BYTES = RB * BLK_BYTES;
    static constexpr int STAGE_ROW = 136;                     // bf16 elements per staged row (128 + padding)
    static constexpr int STAGE_WAVE_BYTES = 2304;             // 8 rows x 272 B, rounded up
    static constexpr int STAGE_BYTES = NW * STAGE_WAVE_BYTES;
    static constexpr int WORK_BYTES = A_RING_BYTES + B_RING_BYTES + STAGE_BYTES;   // + the plan records
    static constexpr int MAX_STEP_DMA = A_PER_WAVE + 2 * COLS_PER_COPIER * 2;      // per copy wave
    static_assert(NP == 4, "four copy waves: one per SIMD");
    static_assert(RB >= 2 * D16_NB && (RB & (RB - 1)) == 0, "the block ring holds one full step; power of two");
    static_assert(RS >= 2 && RS <= 4, "step buffers");
    static_assert((RS - 1) * MAX_STEP_DMA <= 60, "DMA in flight per wave is counted by a 6-bit counter");
    static_assert(WORK_BYTES % 256 == 0, "alignment of the plan records");
};

template <int TRANS, int RS, int RB, int NP>
__global__ __launch_bounds__((8 + NP) * 64) void dds16_kernel(D16Args g) {
    using C = D16Cfg<RS, RB, NP>;
    using E = Elem<bf16_t>;
    constexpr int NBW = C::NBW, NW = C::NW, TM = C::TM, R = D16_REC;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    unsigned char* const a_ring = smem;
    unsigned char* const b_ring = smem + C::A_RING_BYTES;
    int* const s_plan = reinterpret_cast<int*>(smem + C::WORK_BYTES);
    const unsigned lds_a = (unsigned)(uintptr_t)a_ring;
    const unsigned lds_b = (unsigned)(uintptr_t)b_ring;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Workgroup -> (column group, first token tile).  Workgroups are handed to the 8 XCDs round-robin;
    // the workgroups of one XCD cover all column groups of the same few token tiles, so a panel is
    // fetched into that XCD's L2 once and read there by every group.
    const int wg = blockIdx.x;
    const int ng = (wg >> 3) % g.n_groups;
    const int p = (wg & 7) + 8 * ((wg >> 3) / g.n_groups);
    if (p >= g.wg_per_group) return;
    const int ntiles = (g.m_tiles - p + g.wg_per_group - 1) / g.wg_per_group;   // token tiles p, p + P, ...
    const int nb0 = ng * D16_NB;

    // ---- this group's plan records -> LDS ----
    {
        const int4* src = reinterpret_cast<const int4*>(g.plan + (size_t)ng * g.group_ints);
        int4* dst = reinterpret_cast<int4*>(s_plan);
        const int n4 = (2 + g.plan[(size_t)ng * g.group_ints]) * (R / 4);   // header + records + sentinel
        for (int i = tid; i < n4; i += C::NT) dst[i] = src[i];
    }
    __syncthreads();
    const int ns = __builtin_amdgcn_readfirstlane(s_plan[0]);   // steps (k-pairs) per tile
    const int ne = __builtin_amdgcn_readfirstlane(s_plan[1]);   // entries per tile
    const int nsteps = ns * ntiles;                              // global steps of this workgroup
#ifdef PBS_EXP_TIMING
    const bool prof_on = (wg == 100) && (lane == 0) && (wave == 0 || wave == NW);
    const int prof_base = wave == 0 ? 0 : 4096;
#endif
    PBS_T(0);

    // lane l: int l of the record of step s of a tile
    auto fetch_rec = [&](int s) -> int { return s_plan[(1 + s) * R + lane]; };
    // lane d (0..3): entries before the end of global step u + d, where u is step s of tile j
    auto fetch_ends = [&](int j, int s) -> int {
        int sd = s + (lane & 3), jd = j;
        while (sd >= ns) {   // at most once unless a tile has fewer than 4 steps
            sd -= ns;
            ++jd;
        }
        return jd * ne + s_plan[(2 + sd) * R + D16_F_CUM];
    };
    struct Ends {
        int c0, c1, c2, c3;
    };
    auto unpack_ends = [&](Ends& ce, int v) {
        ce.c0 = __builtin_amdgcn_readlane(v, 0);
        ce.c1 = __builtin_amdgcn_readlane(v, 1);
        ce.c2 = RS > 2 ? __builtin_amdgcn_readlane(v, 2) : 0;
        ce.c3 = RS > 3 ? __builtin_amdgcn_readlane(v, 3) : 0;
    };
    // global step t may be issued while u is the oldest unconsumed one (ent_u entries before it) if its
    // panel buffer (t - u < RS) and its block slots (entries of steps u..t <= RB) are free
    auto can_issue = [&](int t, int u, int ent_u, const Ends& ce) -> bool {
        const int d = t - u;
        if (t >= nsteps || d >= RS) return false;
        const int end = d == 0 ? ce.c0 : (d == 1 ? ce.c1 : (d == 2 ? ce.c2 : ce.c3));
        return end - ent_u <= RB;
    };

    const unsigned char* A = static_cast<const unsigned char*>(g.a);
    const unsigned char* D = static_cast<const unsigned char*>(g.data);
    const size_t a_row_bytes = (size_t)g.K * 2;

    // =====================================================================================
    // copy waves
    // =====================================================================================
    if (wave >= NW) {
        if (ns == 0) return;   // no block in this column group: nothing to fetch
        const int dw = wave - NW;
        // panel: instruction q of this wave fills rows (dw*A_PER_WAVE + q)*8 .. +8; lane l serves row l/8,
        // physical chunk l%8, i.e. logical chunk (l%8) ^ swizzle(row)
        int a_row[C::A_PER_WAVE];
        unsigned a_chunk[C::A_PER_WAVE];
#pragma unroll
        for (int q = 0; q < C::A_PER_WAVE; ++q) {
            const int row = (dw * C::A_PER_WAVE + q) * 8 + (lane >> 3);
            a_row[q] = row;
            a_chunk[q] = (unsigned)(((lane & 7) ^ ((row >> 1) & 7)) * 16);
        }
        unsigned b_voff[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if constexpr (TRANS) {
                const int row = q * 16 + (lane >> 2);
                b_voff[q] = row * 64 + (((lane & 3) ^ swz<4>(row)) * 16);
            } else {
                b_voff[q] = q * 1024 + lane * 16;
            }
        }
        // issue the DMA of global step t = step s of tile j (records in vrec); returns the instruction count
        auto issue_step = [&](int t, int j, int vrec) -> int {
            const int m0 = (p + j * g.wg_per_group) * C::BM;
            const int last_row = g.M - 1 - m0;   // rows past the end re-read the last row; never stored
            const int pair = __builtin_amdgcn_readlane(vrec, D16_F_PAIR);
            const unsigned mask = (unsigned)__builtin_amdgcn_readlane(vrec, D16_F_MASK);
            const int base = j * ne + __builtin_amdgcn_readlane(vrec, D16_F_CUM);
            const unsigned char* src = uniform_ptr(A + (size_t)m0 * a_row_bytes + (size_t)pair * C::ROWB);
            const unsigned stage =
                __builtin_amdgcn_readfirstlane(lds_a + (t % RS) * C::PANEL_BYTES + dw * (C::A_PER_WAVE * 1024));
            int n = 0;
#ifndef PBS_EXP_NO_A
#pragma unroll
            for (int q = 0; q < C::A_PER_WAVE; ++q) {
                const int r = a_row[q] < last_row ? a_row[q] : last_row;
                dma16(stage + q * 1024, src, (unsigned)r * (unsigned)a_row_bytes + a_chunk[q]);
            }
            n = C::A_PER_WAVE;
#endif
            // this wave fetches the blocks of columns dw, dw + 4, dw + 8, dw + 12 of both k-blocks
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int c = 0; c < C::COLS_PER_COPIER; ++c) {
                    const int bit = 16 * kk + dw + c * NP;
#ifdef PBS_EXP_NO_B
                    if (false) {
#else
                    if ((mask >> bit) & 1u) {
#endif
                        const int e = base + __popc(mask & ((1u << bit) - 1u));
                        const unsigned char* bsrc =
                            uniform_ptr(D + (size_t)__builtin_amdgcn_readlane(vrec, bit) * C::BLK_BYTES);
                        const unsigned bdst = __builtin_amdgcn_readfirstlane(lds_b + (e & (RB - 1)) * C::BLK_BYTES);
                        dma16(bdst, bsrc, b_voff[0]);
                        dma16(bdst + 1024, bsrc, b_voff[1]);
                        n += 2;
                    }
                }
            }
            return n;
        };

        int pend[RS];   // DMA counts of the issued, not yet consumed steps, oldest first
#pragma unroll
        for (int k = 0; k < RS; ++k) pend[k] = 0;
        int npend = 0;
        auto push = [&](int c) {
#pragma unroll
            for (int k = 0; k < RS; ++k)
                if (npend == k) pend[k] = c;
            ++npend;
        };
        int next = 0, jn = 0, sn = 0;   // next global step to issue = step sn of tile jn
        int vrec = fetch_rec(0);
        auto issue_next = [&]() {
            push(issue_step(next, jn, vrec));
            ++next;
            if (++sn == ns) {
                sn = 0;
                ++jn;
            }
            vrec = fetch_rec(sn);   // consumed at the next issue: the LDS latency is hidden
        };
        Ends ce;
        unpack_ends(ce, fetch_ends(0, 0));
        int ent_u = 0;
        while (can_issue(next, 0, 0, ce)) issue_next();
        int j = 0, s = 0;
        for (int u = 0; u < nsteps; ++u) {
            if (next <= u) {
                // the block ring could not take step u while step u-1 was in use
                drain_barrier();
                issue_next();
            }
            PBS_T(8 + 4 * u + 0);
            const int vends = fetch_ends(j, s);
            int later = 0;   // DMA of the steps after u may stay in flight
#pragma unroll
            for (int k = 1; k < RS; ++k) later += pend[k];
            wait_dma_and_barrier(later);
            PBS_T(8 + 4 * u + 1);
            unpack_ends(ce, vends);
#pragma unroll
            for (int k = 0; k + 1 < RS; ++k) pend[k] = pend[k + 1];
            pend[RS - 1] = 0;
            --npend;
            // every wave is past step u-1 now: its buffers can be refilled
            if (u > 0)
                while (can_issue(next, u, ent_u, ce)) issue_next();
            PBS_T(8 + 4 * u + 2);
            PBS_T(8 + 4 * u + 3);
            ent_u = ce.c0;
            if (++s == ns) {
                s = 0;
                ++j;
            }
        }
        return;
    }

    // =====================================================================================
    // compute waves
    // =====================================================================================
    const int ms = wave & 1;        // token slice (64 tokens)
    const int quarter = wave >> 1;  // 4 block columns
    const int lrow = lane & 31;
    const int h = lane >> 5;

    // Per-lane fragment addresses.  Panel rows are 128 bytes, so the swizzled chunk position only
    // changes address bits 4..6 and the register (bit 4) and k-block (bit 6) selections are XORs with
    // constants; the second token sub-slice is a constant 32 rows further on.
    const int a_lane_off = ((ms * TM) * 32 + lrow) * C::ROWB + (((h * 2) ^ ((lrow >> 1) & 7)) * 16);
    int b_lane_off;
    if constexpr (TRANS) {
        b_lane_off = lrow * 64 + (((h * 2) ^ swz<4>(lrow)) * 16);   // register q: ^ (q * 16)
    } else {
        // transposing 8-byte reads: within 16 lanes, lane s addresses 4 consecutive columns of row s/4
        // and receives, for its own column, the 4 rows as 4 consecutive k
        const int l16 = lane & 15;
        b_lane_off = (16 * h + (l16 >> 2)) * 64 + (((lane >> 4) & 1) * 16 + (l16 & 3) * 4) * 2;
    }
    auto load_a = [&](uint4 (&fa)[TM][2], const unsigned char* panel, int kk) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const unsigned char* pq = panel + (a_lane_off ^ (kk * 64 + q * 16));
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i][q] = *reinterpret_cast<const uint4*>(pq + i * 32 * C::ROWB);
        }
    };
    auto load_b = [&](uint4 (&fb)[2], const unsigned char* pb) {
        if constexpr (TRANS) {
#pragma unroll
            for (int q = 0; q < 2; ++q) fb[q] = *reinterpret_cast<const uint4*>(pb + (b_lane_off ^ (q * 16)));
        } else {
            const unsigned char* pp = pb + b_lane_off;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const uint2 lo = tr16_b64(pp + (8 * q) * 64);
                const uint2 hi = tr16_b64(pp + (8 * q + 4) * 64);
                fb[q] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        }
    };

    bf16_t* out = static_cast<bf16_t*>(g.out);
    const bf16_t* bias = static_cast<const bf16_t*>(g.bias);
    const int col0 = (nb0 + quarter * NBW) * 32;   // first result column of this wave
    bf16_t* stage = reinterpret_cast<bf16_t*>(smem + C::A_RING_BYTES + C::B_RING_BYTES + wave * C::STAGE_WAVE_BYTES);

    f32x16 acc[TM][NBW];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int jc = 0; jc < NBW; ++jc)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][jc][v] = 0.f;
    };
    zero_acc();

    // Stores of one tile: 8 result rows at a time pass through this wave's staging rows so that the
    // global stores are 16 bytes per lane along rows; bias fused.
    auto epilogue = [&](int j) {
        // Everything per-lane is derived again from the lane id behind an opaque copy: hoisted out of the
        // step loop these addresses would stay in registers next to the accumulators and force spills.
        int l = lane;
        asm volatile("" : "+v"(l));
        const int er = l & 31, eh = l >> 5;
        const int m0 = (p + j * g.wg_per_group) * C::BM;
        float bv[NBW];
#pragma unroll
        for (int jc = 0; jc < NBW; ++jc) {
            const int col = col0 + jc * 32 + er;
            bv[jc] = (bias && col < g.N) ? E::to_f32(bias[col]) : 0.f;
        }
        bf16_t* st_w = stage + (4 * eh) * C::STAGE_ROW + er;                    // + vv rows, + jc*32
        const int rd_r = l >> 4, rd_c = (l & 15) * 8;
        const bf16_t* st_r = stage + rd_r * C::STAGE_ROW + rd_c;                // + 4 rows for the second read
        const int col = col0 + rd_c;
#pragma unroll
        for (int t = 0; t < TM; ++t) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
#pragma unroll
                for (int jc = 0; jc < NBW; ++jc)
#pragma unroll
                    for (int vv = 0; vv < 4; ++vv)
                        st_w[vv * C::STAGE_ROW + jc * 32] = E::from_f32(acc[t][jc][4 * gq + vv] + bv[jc]);
#pragma unroll
                for (int pp = 0; pp < 2; ++pp) {
                    const uint4 val = *reinterpret_cast<const uint4*>(st_r + pp * 4 * C::STAGE_ROW);
                    const int row = m0 + (ms * TM + t) * 32 + gq * 8 + pp * 4 + rd_r;
                    if (row < g.M && col < g.N) *reinterpret_cast<uint4*>(out + (size_t)row * g.N + col) = val;
                }
            }
        }
    };

    // same bookkeeping as the copy waves (the barriers must match), without the DMA
    if (ns > 0) {
        int next = 0, ent_u = 0;
        Ends ce;
        unpack_ends(ce, fetch_ends(0, 0));
        while (can_issue(next, 0, 0, ce)) ++next;
        int j = 0, s = 0;
        for (int u = 0; u < nsteps; ++u) {
            if (next <= u) {
                lds_barrier();
                ++next;
            }
            PBS_T(8 + 4 * u + 0);
            const int vends = fetch_ends(j, s);
            const int vrec = fetch_rec(s);
            lds_barrier();
            PBS_T(8 + 4 * u + 1);
            unpack_ends(ce, vends);
            if (u > 0)
                while (can_issue(next, u, ent_u, ce)) ++next;
            ent_u = ce.c0;
            PBS_T(8 + 4 * u + 2);

            // ---- the products of step s ----
            const unsigned mask = (unsigned)__builtin_amdgcn_readlane(vrec, D16_F_MASK);
            const int base = j * ne + __builtin_amdgcn_readlane(vrec, D16_F_CUM);
            const unsigned char* panel = a_ring + (u % RS) * C::PANEL_BYTES;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const unsigned mk = (mask >> (16 * kk)) & 0xffffu;
#ifdef PBS_EXP_NO_COMPUTE
                const unsigned mine = 0;
#else
                const unsigned mine = (mk >> (NBW * quarter)) & ((1u << NBW) - 1u);
#endif
                if (mine == 0) continue;
                int e = base + (kk ? __popc(mask & 0xffffu) : 0) + __popc(mk & ((1u << (NBW * quarter)) - 1u));
                uint4 fa[TM][2];
                load_a(fa, panel, kk);
                // the accumulator index stays static; the branches are wave-uniform
#pragma unroll
                for (int jc = 0; jc < NBW; ++jc) {
                    if ((mine >> jc) & 1u) {
                        uint4 fb[2];
                        load_b(fb, b_ring + (e & (RB - 1)) * C::BLK_BYTES);
                        ++e;
#pragma unroll
                        for (int t = 0; t < TM; ++t) E::mma(acc[t][jc], fa[t], fb);
                    }
                }
            }

            PBS_T(8 + 4 * u + 3);
            if (++s == ns) {
                epilogue(j);
                zero_acc();
                s = 0;
                ++j;
            }
        }
    }
    // a pattern with no block in this group: the result columns are the bias
    if (ns == 0) {
        for (int j = 0; j < ntiles; ++j) epilogue(j);
    }
}

}  // namespace pbs
