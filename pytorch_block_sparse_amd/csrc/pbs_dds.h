// dense x block-sparse -> dense (forward Y = X.W^T and input gradient dX = dY.W).
//
// Work decomposition.  One workgroup owns a BM-token x 8-block-column tile of the result (block
// columns of the *result*: block rows of W for the forward, block columns of W for dX).  Its 8
// compute waves are 4 token slices (TM*32 tokens each) x 2 block-column halves (4 block columns
// each): the two waves of a token slice sit on the same SIMD, so each SIMD sees every block
// product of the tile and the four SIMDs stay balanced however uneven the pattern is, while one
// wave's LDS and scalar work overlaps the other's matrix-core work.
//
// Schedule.  What a tile has to do depends only on the pattern, so it is computed once per pattern
// by dds_plan_kernel and kept in global memory (the "plan"): per group of 8 block columns one
// 64-byte record per k-block that any of them touches (k-block, present-column mask, running entry
// count, the data block of each column).  A workgroup copies its group's records to LDS once.
//
// Data movement.  A step covers SK k-blocks.  Its BM x 32 dense operand panels and its packed
// blocks are copied global -> LDS by the DMA path (global_load_lds_dwordx4, no registers): panels
// into a ring of RS step buffers, blocks into a ring of RB block slots (entry e uses slot e % RB),
// so that RS-1 steps of loads are in flight while one is consumed.  A wave waits for its own DMA
// instructions with an exact s_waitcnt vmcnt(n); one barrier per step publishes the step.
//
// Copy waves.  Issuing a DMA instruction blocks the issuing wave until the texture addresser has
// taken it (about 25 cycles per instruction per CU when all waves stream), so waves that also
// compute would add the copy time to their compute time.  With NP > 0 the workgroup has NP extra
// waves that only issue DMA and wait for it, and the compute waves never touch global memory in
// the main loop.  (fp32 spends 16x longer in the matrix cores per byte and keeps NP = 0.)
//
// LDS layouts (16-byte chunks; a DMA instruction fills 64 consecutive chunks, lane p -> chunk p,
// and each lane may fetch any global address, so the layout is chosen by the addresses):
//   operand panel rows, and packed-block rows when k runs along the row (dX): chunk c of row r
//   sits at chunk position  c ^ swz(r)  of that row -- 16-byte reads of 16 consecutive rows at the
//   same logical chunk then hit 16 distinct bank groups, and the 4 (bf16) or 8 (fp32) lanes that
//   fetch one row still read one contiguous 64/128-byte piece of global memory;
//   packed blocks for the forward stay as stored, [k][n]: bf16 operands are gathered k-major by
//   ds_read_b64_tr_b16, fp32 operands are read one word per k.
#pragma once
#include <type_traits>

#include "pbs_common.h"

namespace pbs {

constexpr int DDS_NB = 8;    // block columns per workgroup tile
constexpr int DDS_NBW = 4;   // block columns per compute wave
constexpr int DDS_NW = 8;    // compute waves per workgroup: 4 token slices x 2 column halves

// ---- plan layout per group of DDS_NB block columns: (KB + 2) records of 16 ints (KB = K/32) ----
//   record 0        header: [0] = nk (present k-blocks), [1] = ne (entries), [2..9] = block column of the
//                   result in each of the group's 8 places, or -1
//   record 1 + i    i-th present k-block: [0..7] data block of each column or -1,
//                   [8] k-block, [9] present-column mask, [10] entries before it
//   record 1 + nk   sentinel: [10] = ne
constexpr int DDS_REC_INTS = 16;
constexpr int DDS_F_KB = 8, DDS_F_MASK = 9, DDS_F_CUM = 10;
constexpr int DDS_H_COL = 2;
static inline size_t dds_plan_group_ints(int KB) { return ((size_t)KB + 2) * DDS_REC_INTS; }

// Which block columns of the result form a group.  Normally group g is columns 8g .. 8g+7.  When the
// per-column block counts are very uneven (largest > 2x the mean) the columns are ranked by count
// and dealt to the half-groups of 4 in serpentine order, so every tile gets about the same number
// of blocks: a tile of a few heavy columns would otherwise run long after all others are done.
// A group may also be given fewer than 8 columns (width), which leaves places empty: more, lighter
// tiles, for launches that would otherwise leave CUs without one.
// slots[8g + j] = block column in place j of group g, or -1.  One workgroup.
constexpr int DDS_BALANCE_MAX_COLS = 4096;
constexpr int DDS_MIN_WIDTH = 5;   // the narrowest group the host asks for
// places of all groups when DDS_BALANCE_MAX_COLS columns are dealt DDS_MIN_WIDTH to a group
constexpr int DDS_SLOT_MAX = DDS_NB * ((DDS_BALANCE_MAX_COLS + DDS_MIN_WIDTH - 1) / DDS_MIN_WIDTH);
__global__ __launch_bounds__(256) void dds_slots_kernel(const int32_t* __restrict__ ptr, int nblk_n, int n_groups,
                                                        int width, int* slots) {
    constexpr int NT = 256;
    __shared__ int s_cnt[DDS_BALANCE_MAX_COLS];
    __shared__ int s_slot[DDS_SLOT_MAX];
    __shared__ int s_max, s_sum;
    const int tid = threadIdx.x;
    const int total = n_groups * DDS_NB;
    bool skewed = false;
    // (a table that would not fit s_slot keeps the natural order)
    if (nblk_n <= DDS_BALANCE_MAX_COLS && n_groups >= 2 && total <= DDS_SLOT_MAX) {
        if (tid == 0) {
            s_max = 0;
            s_sum = 0;
        }
        __syncthreads();
        for (int c = tid; c < nblk_n; c += NT) {
            const int n = ptr[c + 1] - ptr[c];
            s_cnt[c] = n;
            atomicMax(&s_max, n);
            atomicAdd(&s_sum, n);
        }
        __syncthreads();
        skewed = (long long)s_max * nblk_n > 2ll * s_sum;
    }
    if (!skewed) {
        // group g holds columns g * width .. + width - 1; with fewer than 8 they alternate between the two
        // halves of the group's places, so that tiles of 4 places and the column halves of the waves get
        // equal shares
        for (int i = tid; i < total; i += NT) {
            const int j = i % DDS_NB;
            const int l = width == DDS_NB ? j : (j < 4 ? 2 * j : 2 * (j - 4) + 1);
            const int c = (i / DDS_NB) * width + l;
            slots[i] = (l < width && c < nblk_n) ? c : -1;
        }
        return;
    }
    for (int i = tid; i < total; i += NT) s_slot[i] = -1;
    __syncthreads();
    const int units = 2 * n_groups;   // half-groups of 4 columns
    for (int c = tid; c < nblk_n; c += NT) {
        const int n = s_cnt[c];
        int rank = 0;
        for (int o = 0; o < nblk_n; ++o) {
            const int m = s_cnt[o];
            rank += (m > n || (m == n && o < c)) ? 1 : 0;
        }
        const int place = rank / units;            // 0..3 within the half-group
        int u = rank % units;
        if (place & 1) u = units - 1 - u;          // serpentine: heavy and light columns pair up
        s_slot[(u >> 1) * DDS_NB + (u & 1) * 4 + place] = c;
    }
    __syncthreads();
    for (int i = tid; i < total; i += NT) slots[i] = s_slot[i];
}

// One workgroup per group of 8 block columns merges their sorted block lists.
__global__ __launch_bounds__(256) void dds_plan_kernel(const int32_t* __restrict__ ptr, const int32_t* __restrict__ idx,
                                                       const int* __restrict__ slots, int nblk_n, int KB, int nnz,
                                                       int* plan, int group_ints) {
    constexpr int NB = DDS_NB, SEG = 128, NT = 256, R = DDS_REC_INTS;
    __shared__ int s_tbl[SEG * NB];
    __shared__ int s_lo[NB], s_hi[NB], s_col[NB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int* out = plan + (size_t)blockIdx.x * group_ints;
    int* rec = out + R;
    if (tid < NB) {
        const int c = slots[blockIdx.x * NB + tid];
        const bool ok = c >= 0 && c < nblk_n;
        s_col[tid] = ok ? c : -1;
        s_lo[tid] = ok ? clamp_entry(ptr[c], nnz) : 0;
        s_hi[tid] = ok ? clamp_entry(ptr[c + 1], nnz) : 0;
    }
    __syncthreads();
    int nk = 0, ne = 0;   // running totals (kept by every thread of wave 0)
    for (int seg0 = 0; seg0 < KB; seg0 += SEG) {
        for (int i = tid; i < SEG * NB; i += NT) s_tbl[i] = -1;
        __syncthreads();
        for (int jc = 0; jc < NB; ++jc) {
            for (int e = s_lo[jc] + tid; e < s_hi[jc]; e += NT) {
                const int kb = idx[2 * e] - seg0;
                const int b = idx[2 * e + 1];
                if (kb >= 0 && kb < SEG && kb + seg0 < KB && b >= 0 && b < nnz) s_tbl[kb * NB + jc] = b;
            }
        }
        __syncthreads();
        if (wave == 0) {
            for (int base = 0; base < SEG; base += 64) {
                const int kbl = base + lane;
                int present = 0;
#pragma unroll
                for (int j = 0; j < NB; ++j) present |= (s_tbl[kbl * NB + j] >= 0) ? (1 << j) : 0;
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
                    int* r = rec + (size_t)(nk + __popcll(m & ((1ull << lane) - 1ull))) * R;
#pragma unroll
                    for (int j = 0; j < NB; ++j) r[j] = s_tbl[kbl * NB + j];
                    r[DDS_F_KB] = seg0 + kbl;
                    r[DDS_F_MASK] = present;
                    r[DDS_F_CUM] = ne + incl - cnt;
#pragma unroll
                    for (int j = DDS_F_CUM + 1; j < R; ++j) r[j] = 0;
                }
                nk += __popcll(m);
                ne += total;
            }
        }
        __syncthreads();
    }
    if (wave == 0 && lane < R) {
        // header: counts, then the block column in each of the group's 8 places
        int hv = 0;
        if (lane == 0) hv = nk;
        else if (lane == 1) hv = ne;
        else if (lane >= DDS_H_COL && lane < DDS_H_COL + NB) hv = s_col[lane - DDS_H_COL];
        out[lane] = hv;
        int* r = rec + (size_t)nk * R;   // sentinel
        r[lane] = lane < NB ? -1 : (lane == DDS_F_CUM ? ne : 0);
    }
}


struct DdsArgs {
    const void* a;         // [M, K] row-major
    const void* data;      // [nnz*32, 32]
    const int* plan;       // built by dds_plan_kernel for this pattern and direction
    const void* bias;      // nullptr or [N]
    void* out;             // [M, N] row-major
    int M, N, K, nnz;
    int m_tiles, n_groups, group_ints;
};

// TRANS = 0: B[k][n] = block[k*32 + n]   (forward: the packed block is W_block^T = [in][out])
// TRANS = 1: B[k][n] = block[n*32 + k]   (dX: contraction runs along the packed block's rows)
template <typename T, int TRANS, int TM, int SK, int RS, int RB, int NP, int NBW_ = DDS_NBW, int NSL_ = 4>
struct DdsCfg {
    using E = Elem<T>;
    static constexpr int NW = DDS_NW;                    // compute waves
    // The 8 compute waves are NSL token slices x NH = 8 / NSL column parts of NBW block columns each:
    //   NSL = 4, NBW = 4   the tile covers its whole group of 8 block columns (two halves);
    //   NSL = 4, NBW = 2   the tile covers half a group: twice as many, half as wide tiles;
    //   NSL = 8, NBW = 8   every wave has all 8 block columns and its own 32 * TM tokens: all waves do
    //                      the same products, so the barrier per step costs nothing however uneven the
    //                      pattern is (with column halves a step lasts as long as its fuller half).
    static constexpr int NBW = NBW_;
    static constexpr int NSL = NSL_;
    static constexpr int NH = DDS_NW / NSL_;
    static constexpr int TILE_COLS = NH * NBW_;          // block columns per tile
    static constexpr int NSUB = DDS_NB / TILE_COLS;      // tiles per column group
    static_assert((NSL_ == 4 && (NBW_ == 4 || NBW_ == 2)) || (NSL_ == 8 && NBW_ == 8), "wave layout");
    static constexpr int ND = NP ? NP : NW;              // waves that issue DMA
    static constexpr int NT = (NW + NP) * 64;
    static constexpr int BM = NSL_ * TM * 32;
    static constexpr int ROWB = 32 * E::ESZ;             // bytes of one 32-wide operand row
    static constexpr int CPR = ROWB / 16;                // 16-byte chunks per row (4 or 8)
    static constexpr int RPI = 64 / CPR;                 // rows filled by one DMA instruction (16 or 8)
    static constexpr int PANEL_BYTES = BM * ROWB;        // one k-block of the dense operand
    static constexpr int PANEL_INSTR = PANEL_BYTES / 1024;
    static constexpr int A_PER_WAVE = PANEL_INSTR / ND;  // DMA instructions per issuing wave per k-block
    static constexpr int COLS_PER_COPIER = DDS_NB / ND;  // block columns whose blocks a copy wave fetches
    static constexpr int STEP_BYTES = SK * PANEL_BYTES;
    static constexpr int BLK_BYTES = 1024 * E::ESZ;
    static constexpr int BLK_INSTR = BLK_BYTES / 1024;   // DMA instructions per packed block (2 or 4)
    static constexpr int A_RING_BYTES = RS * STEP_BYTES;
    static constexpr int B_RING_BYTES = RB * BLK_BYTES;
    static constexpr int RING_BYTES = A_RING_BYTES + B_RING_BYTES;
    // the epilogue stages 8 result rows of a compute wave's columns at a time through LDS (rows padded by
    // 16 bytes: the two lane halves write rows 4 apart, which would otherwise meet in the same banks)
    static constexpr int EPI_ROW_BYTES = NBW_ * 32 * E::ESZ + 16;
    static constexpr int EPI_WAVE_BYTES = 8 * EPI_ROW_BYTES;
    static constexpr int EPI_BYTES = NW * EPI_WAVE_BYTES;
    static constexpr int WORK_BYTES = RING_BYTES > EPI_BYTES ? RING_BYTES : EPI_BYTES;   // + the plan records
    static_assert(PANEL_INSTR % ND == 0 && A_PER_WAVE >= 1, "panel DMA must divide evenly over the issuing waves");
    static_assert(DDS_NB % ND == 0 && COLS_PER_COPIER >= 1, "block columns must divide evenly over the issuing waves");
    static_assert(RS >= 2, "need at least two step buffers");
    static_assert(RB >= SK * DDS_NB && (RB & (RB - 1)) == 0, "the block ring holds one full step; power of two");
    static_assert(WORK_BYTES % 16 == 0, "alignment of the plan records");
};

// chunk swizzle of a row: bf16 rows have 4 chunks, fp32 rows 8
template <int CPR>
static __device__ __forceinline__ int swz(int r) {
    return CPR == 4 ? ((r >> 2) & 3) : ((r >> 1) & 7);
}

template <typename T, int TRANS, int TM, int SK, int RS, int RB, int NP, int NBW_ = DDS_NBW, int NSL_ = 4>
__global__ __launch_bounds__((DDS_NW + NP) * 64) void dds_kernel(DdsArgs g) {
    using C = DdsCfg<T, TRANS, TM, SK, RS, RB, NP, NBW_, NSL_>;
    using E = typename C::E;
    constexpr int NBW = C::NBW, NW = DDS_NW, ND = C::ND, NQ = E::NQ, CPR = C::CPR, R = DDS_REC_INTS;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    unsigned char* const a_ring = smem;
    unsigned char* const b_ring = smem + C::A_RING_BYTES;
    int* const s_plan = reinterpret_cast<int*>(smem + C::WORK_BYTES);   // this group's records
    const unsigned lds_a = (unsigned)(uintptr_t)a_ring;
    const unsigned lds_b = (unsigned)(uintptr_t)b_ring;

    const int n_cols = g.n_groups * C::NSUB;   // tiles along the result columns
    const int tile = xcd_tile_id(blockIdx.x, g.m_tiles * n_cols);
    if (tile < 0) return;
    // Order of the tiles inside an XCD's range: blocks of 4 token tiles x 8 column tiles, so that the
    // 32 workgroups an XCD runs at a time share 4 operand panels and 8 groups of weight blocks in
    // its L2 (token-tile-major order would stream all the weights through every XCD's L2).
    int mt, nc;
    if ((n_cols % 8) == 0 && (g.m_tiles % 4) == 0) {
        const int blk = tile >> 5, within = tile & 31;
        const int ncb = blk % (n_cols / 8), mtb = blk / (n_cols / 8);
        mt = mtb * 4 + (within >> 3);
        nc = ncb * 8 + (within & 7);
    } else {
        mt = tile / n_cols;
        nc = tile % n_cols;
    }
    const int ng = nc / C::NSUB;                        // column group (plan records)
    const int col_lo = (nc % C::NSUB) * C::TILE_COLS;   // first of this tile's columns within the group
    const int m0 = mt * C::BM;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- this group's plan records -> LDS ----
    {
        const int4* src = reinterpret_cast<const int4*>(g.plan + (size_t)ng * g.group_ints);
        int4* dst = reinterpret_cast<int4*>(s_plan);
        const int n4 = (2 + g.plan[(size_t)ng * g.group_ints]) * (R / 4);   // header + nk records + sentinel
        for (int i = tid; i < n4; i += C::NT) dst[i] = src[i];
    }
    __syncthreads();
    const int nk = __builtin_amdgcn_readfirstlane(s_plan[0]);
    const int ns = (nk + SK - 1) / SK;
    // Plan fields are read a whole step at a time: lane l of fetch_recs(t) holds int (l % 16) of the
    // (l / 16)-th k-block record of step t (records past the last one read the sentinel), and single
    // fields are then picked with v_readlane -- one LDS round trip per step instead of one per field.
    auto kend = [&](int s) -> int { const int i = (s + 1) * SK; return i < nk ? i : nk; };
    auto fetch_recs = [&](int t) -> int {
        int i = t * SK + (lane >> 4);
        if (i > nk) i = nk;
        return s_plan[(1 + i) * R + (lane & 15)];
    };
    auto field = [&](int vrec, int k, int f) -> int { return __builtin_amdgcn_readlane(vrec, k * R + f); };

    // Bookkeeping shared by all waves.  ce.c<d> = entries before the end of step s + d; step t may be
    // issued while step s is the oldest unconsumed one if its panel buffer (t - s < RS) and its block
    // slots (entries of steps s..t <= RB) are free.
    struct Ends {
        int c0, c1, c2, c3;   // scalars on purpose: an indexed array would go to scratch memory
    };
    static_assert(RS <= 4, "Ends holds four step ends");
    static_assert(SK * R <= 64, "one lane per record int of a step");
    auto fetch_ends = [&](int s) -> int {   // lane d: entries before the end of step s + d
        int i = (s + (lane & 3) + 1) * SK;
        if (i > nk) i = nk;
        return s_plan[(1 + i) * R + DDS_F_CUM];
    };
    auto unpack_ends = [&](Ends& ce, int v) {
        ce.c0 = __builtin_amdgcn_readlane(v, 0);
        ce.c1 = RS > 1 ? __builtin_amdgcn_readlane(v, 1) : 0;
        ce.c2 = RS > 2 ? __builtin_amdgcn_readlane(v, 2) : 0;
        ce.c3 = RS > 3 ? __builtin_amdgcn_readlane(v, 3) : 0;
    };
    auto can_issue = [&](int t, int s, int cum_s, const Ends& ce) -> bool {
        const int d = t - s;
        if (t >= ns || d >= RS) return false;
        const int end = d == 0 ? ce.c0 : (d == 1 ? ce.c1 : (d == 2 ? ce.c2 : ce.c3));
        return end - cum_s <= RB;
    };

    const unsigned char* A_tile = static_cast<const unsigned char*>(g.a) + (size_t)m0 * g.K * E::ESZ;
    const unsigned char* D = static_cast<const unsigned char*>(g.data);

    // =====================================================================================
    // copy side: issue the DMA of step t; returns how many DMA instructions this wave issued
    // =====================================================================================
    struct Issuer {
        unsigned a_voff[C::A_PER_WAVE];
        unsigned b_voff[C::BLK_INSTR];
    };
    auto make_issuer = [&](int dw) -> Issuer {
        // panel: copy wave dw fills instructions dw*A_PER_WAVE + i of every k-block; lane p of instruction
        // q serves row q*RPI + p/CPR and physical chunk p%CPR, i.e. logical chunk (p%CPR) ^ swz(row)
        Issuer is;
#pragma unroll
        for (int i = 0; i < C::A_PER_WAVE; ++i) {
            const int q = dw * C::A_PER_WAVE + i;
            const int row = q * C::RPI + lane / CPR;
            const int chunk = (lane % CPR) ^ swz<CPR>(row);
            int r = row;
            if (m0 + r >= g.M) r = g.M - 1 - m0;   // rows past the end re-read the last row; never stored
            is.a_voff[i] = (unsigned)r * (unsigned)(g.K * E::ESZ) + chunk * 16;
        }
        // packed block: instruction q of a block; forward keeps the block as stored, dX swizzles rows
#pragma unroll
        for (int q = 0; q < C::BLK_INSTR; ++q) {
            if constexpr (TRANS) {
                const int row = q * C::RPI + lane / CPR;
                is.b_voff[q] = row * C::ROWB + ((lane % CPR) ^ swz<CPR>(row)) * 16;
            } else {
                is.b_voff[q] = q * 1024 + lane * 16;
            }
        }
        return is;
    };
    auto issue_step = [&](const Issuer& is, int dw, int t, int vrec) -> int {
        const int cnt = kend(t) - t * SK;   // k-blocks of this step
        const unsigned stage = lds_a + (t % RS) * C::STEP_BYTES + dw * (C::A_PER_WAVE * 1024);
        int n = 0;
#pragma unroll
        for (int k = 0; k < SK; ++k) {
            if (k < cnt) {
                const unsigned char* src = uniform_ptr(A_tile + (size_t)field(vrec, k, DDS_F_KB) * C::ROWB);
                const unsigned dst = __builtin_amdgcn_readfirstlane(stage + k * C::PANEL_BYTES);
#pragma unroll
                for (int q = 0; q < C::A_PER_WAVE; ++q) dma16(dst + q * 1024, src, is.a_voff[q]);
                n += C::A_PER_WAVE;
                // this wave fetches the blocks of columns dw, dw + ND, ...
                const int mask = field(vrec, k, DDS_F_MASK);
                const int base = field(vrec, k, DDS_F_CUM);
#pragma unroll
                for (int c = 0; c < C::COLS_PER_COPIER; ++c) {
                    const int j = dw + c * ND;
                    if (((mask >> j) & 1) && (C::NSUB == 1 || (j >= col_lo && j < col_lo + C::TILE_COLS))) {
                        const int e = base + __popc(mask & ((1 << j) - 1));
                        const unsigned char* bsrc =
                            uniform_ptr(D + (size_t)__builtin_amdgcn_readlane(vrec, k * R + j) * C::BLK_BYTES);
                        const unsigned bdst = __builtin_amdgcn_readfirstlane(lds_b + (e & (RB - 1)) * C::BLK_BYTES);
#pragma unroll
                        for (int q = 0; q < C::BLK_INSTR; ++q) dma16(bdst + q * 1024, bsrc, is.b_voff[q]);
                        n += C::BLK_INSTR;
                    }
                }
            }
        }
        return n;
    };

    // the step loop of a wave that copies (and, with NP == 0, also computes through `compute`)
    auto copy_loop = [&](int dw, auto&& compute) {
        const Issuer is = make_issuer(dw);
        int pend[RS];   // DMA counts of the issued, not yet consumed steps, oldest first
#pragma unroll
        for (int k = 0; k < RS; ++k) pend[k] = 0;
        int npend = 0, next = 0, cum_s = 0;
        auto push = [&](int c) {
#pragma unroll
            for (int k = 0; k < RS; ++k)
                if (npend == k) pend[k] = c;
            ++npend;
        };
        Ends ce;
        unpack_ends(ce, fetch_ends(0));
        int vrec = fetch_recs(0);   // records of step `next`, fetched one issue ahead
        while (can_issue(next, 0, 0, ce)) {
            push(issue_step(is, dw, next, vrec));
            ++next;
            vrec = fetch_recs(next);
        }
        for (int s = 0; s < ns; ++s) {
            if (next <= s) {
                // the block ring could not take step s while step s-1 was in use
                drain_barrier();
                push(issue_step(is, dw, s, vrec));
                next = s + 1;
                vrec = fetch_recs(next);
            }
            const int vends = fetch_ends(s);
            int later = 0;   // DMA of the steps after s may stay in flight
#pragma unroll
            for (int k = 1; k < RS; ++k) later += pend[k];
            wait_dma_and_barrier(later);
            unpack_ends(ce, vends);
#pragma unroll
            for (int k = 0; k + 1 < RS; ++k) pend[k] = pend[k + 1];
            pend[RS - 1] = 0;
            --npend;
            // every wave is past step s-1 now: its buffers can be refilled
            if (s > 0)
                while (can_issue(next, s, cum_s, ce)) {
                    push(issue_step(is, dw, next, vrec));
                    ++next;
                    vrec = fetch_recs(next);
                }
            compute(s);
            cum_s = ce.c0;
        }
        drain_barrier();   // the rings are reused by the epilogue
    };

    if constexpr (NP > 0) {
        if (wave >= NW) {
            copy_loop(wave - NW, [](int) {});
            return;
        }
    }

    // =====================================================================================
    // compute side
    // =====================================================================================
    const int ms = wave % C::NSL;       // token slice
    const int half = wave / C::NSL;     // block-column part of the tile
    const int col_w = col_lo + half * NBW;   // first of this wave's columns within the group
    const int lrow = lane & 31;
    const int h = lane >> 5;

    f32x16 acc[TM][NBW];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < NBW; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // per-lane offsets of the fragment reads
    int a_frag_off[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) a_frag_off[i] = ((ms * TM + i) * 32 + lrow) * C::ROWB;
    const int a_sw = swz<CPR>(lrow);   // (ms*TM+i)*32 is a multiple of 32: the swizzle depends on lrow only
    int b_frag_off;
    if constexpr (TRANS) {
        b_frag_off = lrow * C::ROWB;   // + ((h*NQ+q) ^ swz(lrow)) * 16
    } else if constexpr (E::ESZ == 4) {
        b_frag_off = ((16 * h) * 32 + lrow) * 4;
    } else {
        // transposing 8-byte reads: within 16 lanes, lane s addresses 4 consecutive columns of row s/4
        // and receives, for its own column, the 4 rows as 4 consecutive k
        const int l16 = lane & 15;
        b_frag_off = (16 * h + (l16 >> 2)) * 64 + (((lane >> 4) & 1) * 16 + (l16 & 3) * 4) * 2;
    }
    int chunk_off[NQ];   // swizzled chunk offsets of this lane's k range, shared by panel rows and dX block rows
#pragma unroll
    for (int q = 0; q < NQ; ++q) chunk_off[q] = ((h * NQ + q) ^ a_sw) * 16;

    auto load_a = [&](uint4 (&fa)[TM][NQ], const unsigned char* panel) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < NQ; ++q) fa[i][q] = *reinterpret_cast<const uint4*>(panel + a_frag_off[i] + chunk_off[q]);
    };
    auto load_b = [&](uint4 (&fb)[NQ], const unsigned char* pb) {
        if constexpr (TRANS) {
            const unsigned char* p = pb + b_frag_off;
#pragma unroll
            for (int q = 0; q < NQ; ++q) fb[q] = *reinterpret_cast<const uint4*>(p + chunk_off[q]);
        } else if constexpr (E::ESZ == 4) {
            const uint32_t* p = reinterpret_cast<const uint32_t*>(pb + b_frag_off);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                fb[q].x = p[(4 * q + 0) * 32];
                fb[q].y = p[(4 * q + 1) * 32];
                fb[q].z = p[(4 * q + 2) * 32];
                fb[q].w = p[(4 * q + 3) * 32];
            }
        } else {
            const unsigned char* p = pb + b_frag_off;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const uint2 lo = tr16_b64(p + (8 * q) * 64);
                const uint2 hi = tr16_b64(p + (8 * q + 4) * 64);
                fb[q] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        }
    };
    // (mask, entries before) of the k-blocks of the current step, read ahead of the barrier
    int st_mask[SK], st_cum[SK];
    auto load_step_recs = [&](int s) {
        const int v = fetch_recs(s);
#pragma unroll
        for (int k = 0; k < SK; ++k) {
            st_mask[k] = s * SK + k < nk ? field(v, k, DDS_F_MASK) : 0;
            st_cum[k] = field(v, k, DDS_F_CUM);
        }
    };
    auto compute_step = [&](int s) {
        const unsigned char* stage = a_ring + (s % RS) * C::STEP_BYTES;
#pragma unroll
        for (int k = 0; k < SK; ++k) {
            const int mask = st_mask[k];
            const int mine = (mask >> col_w) & ((1 << NBW) - 1);
            if (mine == 0) continue;
            int e = st_cum[k] + __popc(mask & ((1 << col_w) - 1));
            uint4 fa[TM][NQ];
            load_a(fa, stage + k * C::PANEL_BYTES);
            // the accumulator index stays static; the branches are wave-uniform
#pragma unroll
            for (int j = 0; j < NBW; ++j) {
                if ((mine >> j) & 1) {
                    uint4 fb[NQ];
                    load_b(fb, b_ring + (e & (RB - 1)) * C::BLK_BYTES);
                    ++e;
#pragma unroll
                    for (int t = 0; t < TM; ++t) E::mma(acc[t][j], fa[t], fb);
                }
            }
        }
    };

    if constexpr (NP == 0) {
        copy_loop(wave, [&](int s) {
            load_step_recs(s);
            compute_step(s);
        });
    } else {
        // same bookkeeping as the copy waves (the barriers must match), without the DMA
        int next = 0, cum_s = 0;
        Ends ce;
        unpack_ends(ce, fetch_ends(0));
        while (can_issue(next, 0, 0, ce)) ++next;
        for (int s = 0; s < ns; ++s) {
            if (next <= s) {
                lds_barrier();
                next = s + 1;
            }
            const int vends = fetch_ends(s);
            load_step_recs(s);
            lds_barrier();
            unpack_ends(ce, vends);
            if (s > 0)
                while (can_issue(next, s, cum_s, ce)) ++next;
            compute_step(s);
            cum_s = ce.c0;
        }
        lds_barrier();
    }

    // ---- epilogue: each wave passes its results, 8 rows at a time, through its own LDS region (inside the
    //      rings, which are idle now) so that the global stores are 16 bytes per lane along rows; bias fused ----
    T* out = static_cast<T*>(g.out);
    const T* bias = static_cast<const T*>(g.bias);
    unsigned char* epi = smem + wave * C::EPI_WAVE_BYTES;
    int colid[NBW];   // block columns of the result this wave owns (-1: none)
#pragma unroll
    for (int j = 0; j < NBW; ++j) colid[j] = __builtin_amdgcn_readfirstlane(s_plan[DDS_H_COL + col_w + j]);
    float bv[NBW];
#pragma unroll
    for (int j = 0; j < NBW; ++j) {
        bv[j] = (bias && colid[j] >= 0) ? E::to_f32(bias[colid[j] * 32 + lrow]) : 0.f;
    }
    constexpr int EPL = 16 / E::ESZ;                       // elements per 16-byte chunk
    constexpr int WCOLS = NBW * 32;                        // result columns of one wave
    constexpr int CHUNKS_PER_ROW = WCOLS / EPL;            // 16-byte chunks per staged row
    constexpr int ROWS_PER_PASS = 64 / CHUNKS_PER_ROW;     // rows stored by one wave instruction
    constexpr int PASSES = 8 / ROWS_PER_PASS;              // store instructions per 8 staged rows
    static_assert(ROWS_PER_PASS >= 1 && 8 % ROWS_PER_PASS == 0, "8 staged rows are stored in whole passes");
    const int rd_r = lane / CHUNKS_PER_ROW, rd_c = (lane % CHUNKS_PER_ROW) * EPL;
    int cid = colid[0];   // the block column this lane's chunk belongs to
#pragma unroll
    for (int j = 1; j < NBW; ++j) cid = (rd_c >= j * 32) ? colid[j] : cid;
    const int col = cid * 32 + (rd_c & 31);
#pragma unroll
    for (int t = 0; t < TM; ++t) {
        const int rbase = m0 + (ms * TM + t) * 32;
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {   // rows 8 gq .. 8 gq + 7 of the 32
#pragma unroll
            for (int j = 0; j < NBW; ++j)
#pragma unroll
                for (int vv = 0; vv < 4; ++vv)
                    *reinterpret_cast<T*>(epi + (4 * h + vv) * C::EPI_ROW_BYTES + (j * 32 + lrow) * E::ESZ) =
                        E::from_f32(acc[t][j][4 * gq + vv] + bv[j]);
            uint4 val[PASSES];   // all reads first: one wait for the staged rows
#pragma unroll
            for (int p = 0; p < PASSES; ++p)
                val[p] = *reinterpret_cast<const uint4*>(epi + (p * ROWS_PER_PASS + rd_r) * C::EPI_ROW_BYTES + rd_c * E::ESZ);
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const int row = rbase + gq * 8 + p * ROWS_PER_PASS + rd_r;
                if (row < g.M && cid >= 0) *reinterpret_cast<uint4*>(out + (size_t)row * g.N + col) = val[p];
            }
        }
    }
}

}  // namespace pbs
