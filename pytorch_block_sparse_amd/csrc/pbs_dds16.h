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
// LDS) and walks several token tiles; the stream of steps simply continues across tile boundaries.
//
// No barriers in the step loop.  With a barrier per step all waves of a SIMD do their bookkeeping at
// the same time and their matrix work at the same time, so the matrix cores idle during the former,
// and every step lasts as long as its slowest wave (the pattern gives the waves different numbers of
// blocks).  Instead the 4 copy waves and the 8 compute waves run as producers and consumers of the
// two rings and publish their progress in LDS words:
//   landed[c]   steps whose DMA from copy wave c has arrived, modulo 256.  The copy wave does not wait
//               for its loads: after the loads of step t it issues one more DMA that copies the number
//               (t + 1) % 256 from a table in global memory onto landed[c]; a wave's loads complete in
//               order, so the number appears when the step's operands are in place;
//   done[w]     (steps, block entries) compute wave w has finished reading.
// A compute wave starts step u when every landed[c] has reached u + 1; a copy wave issues step t when every
// done[w].steps >= t - RS + 1 (panel buffer free) and entries_end(t) - min done[w].entries <= RB
// (block slots free).  All counters only grow, each has one writer, and waves poll with s_sleep, so
// waves drift apart by up to the ring depth and one wave's overhead overlaps another's matrix work.
//
// Plan (built by dds16_plan_kernel per pattern and direction): per group of 16 block columns, one
// 256-byte record per k-pair that any of them touches:
//   [0..31]  data blocks of the pair's entries, in entry order (unused places hold -1)
//   [32] k-pair index   [33] presence mask (bit 16*odd + column)   [34] entries before this pair
// preceded by a header record ([0] = pairs present, [1] = entries) and followed by a sentinel
// ([34] = entries).  The entries of a pair are its present (k-block, column) positions in mask-bit
// order: even k-block first, columns ascending.  Entry e lives in block slot e % RB.
//
// LDS: [A ring: RS steps x 16 KB][block ring: RB x 2 KB][epilogue staging: 8 x 2304 B][progress words][plan records].
// Panel rows are 128 bytes (8 chunks of 16 bytes); chunk c of row r sits at position c ^ ((r >> 1) & 7),
// which makes the 16-byte fragment reads of 16 consecutive rows conflict-free.  Packed blocks are laid
// out as in the narrow kernel (pbs_dds.h).
#pragma once
#include "pbs_common.h"
#include "pbs_dds.h"

namespace pbs {

#ifndef D16_SLEEP
#define D16_SLEEP 1
#endif
constexpr int D16_NB = 16;      // block columns per tile
constexpr int D16_REC = 64;     // ints per plan record
constexpr int D16_F_PAIR = 32, D16_F_MASK = 33, D16_F_CUM = 34;
constexpr int D16_BM = 128;     // tokens per tile
static inline size_t dds16_plan_group_ints(int KB) { return ((size_t)(KB / 2) + 2) * D16_REC; }
constexpr int D16_SEQ_INTS = 256;   // table 0..255 behind the plan records: source of the progress DMA

// One workgroup per group of 16 block columns merges their sorted block lists into k-pair records.
__global__ __launch_bounds__(256) void dds16_plan_kernel(const int32_t* __restrict__ ptr, const int32_t* __restrict__ idx,
                                                         int nblk_n, int KB, int nnz, int* plan, int group_ints, int* seq) {
    constexpr int NB = D16_NB, SEG = 128, NT = 256, R = D16_REC;
    __shared__ int s_tbl[SEG * NB];
    __shared__ int s_ptr[NB + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nb0 = blockIdx.x * NB;
    int* out = plan + (size_t)blockIdx.x * group_ints;
    int* rec = out + R;
    if (tid <= NB) {
        const int nb = nb0 + tid;
        s_ptr[tid] = clamp_entry(ptr[nb < nblk_n ? nb : nblk_n], nnz);
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
                int n = 0;
#pragma unroll
                for (int j = 0; j < 2 * NB; ++j) {
                    const int b = s_tbl[lane * 2 * NB + j];
                    if (b >= 0) r[n++] = b;
                }
                for (; n < 2 * NB; ++n) r[n] = -1;
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
    if (blockIdx.x == 0) seq[tid] = tid;   // the numbers the copy waves publish their progress with
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
    const int* seq;        // the table 0..255 written by dds16_plan_kernel
    const void* bias;      // nullptr or [N]
    void* out;             // [M, N] row-major
    int M, N, K, nnz;
    int m_tiles, n_groups, group_ints;
    int wg_per_group;      // workgroups that share the token tiles of one column group
};

template <int TM_, int RS, int RB, int NP>
struct D16Cfg {
    // 8 compute waves = (4 / TM) token slices of TM * 32 tokens x (2 * TM) column groups of NBW = 8 / TM block
    // columns; wave w has slice w % (4 / TM), so the waves that share a SIMD (w, w + 4) share their slice
    static constexpr int NW = 8, NT = (NW + NP) * 64, BM = D16_BM, TM = TM_, NBW = 8 / TM_, NSL = 4 / TM_;
    static_assert(TM_ == 1 || TM_ == 2 || TM_ == 4, "token sub-slices per wave");
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
    // progress words: done steps [NW][64] then done entries [NW][64] (every lane of a compute wave writes
    // its own copy, lane 0's is read), then landed [NP][64] (the progress DMA writes one copy per lane)
    static constexpr int DONE_BYTES = NW * 64 * 8;
    static constexpr int FLAG_BYTES = DONE_BYTES + NP * 256 + 256;   // landed[c]: 64 copies of one word per copy wave; failure word
    static constexpr int FLAG_OFF = A_RING_BYTES + B_RING_BYTES + STAGE_BYTES;
    static constexpr int WORK_BYTES = FLAG_OFF + FLAG_BYTES;   // + the plan records
    static constexpr int SPIN_LIMIT = 1 << 20;                // polls before a wave gives up waiting
    static constexpr int MAX_STEP_DMA = A_PER_WAVE + 2 * COLS_PER_COPIER * 2;      // per copy wave
    static_assert(NP == 4, "four copy waves: one per SIMD");
    static_assert(RB >= 2 * D16_NB && (RB & (RB - 1)) == 0, "the block ring holds one full step; power of two");
    static_assert(RS >= 2 && RS <= 4, "step buffers");
    static_assert((RS - 1) * MAX_STEP_DMA <= 60, "DMA in flight per wave is counted by a 6-bit counter");
    static_assert(WORK_BYTES % 256 == 0, "alignment of the plan records");
};

template <int TRANS, int TM_, int RS, int RB, int NP>
__global__ __launch_bounds__((8 + NP) * 64) void dds16_kernel(D16Args g) {
    using C = D16Cfg<TM_, RS, RB, NP>;
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

    // ---- this group's plan records -> LDS; progress words start at zero ----
    int* const s_done = reinterpret_cast<int*>(smem + C::FLAG_OFF);                     // [2][NW][64]
    int* const s_landed = reinterpret_cast<int*>(smem + C::FLAG_OFF + C::DONE_BYTES);   // [NP]
    int* const s_fail = s_landed + NP * 64;   // set by a copy wave whose wait ran into its bound
    {
        const int4* src = reinterpret_cast<const int4*>(g.plan + (size_t)ng * g.group_ints);
        int4* dst = reinterpret_cast<int4*>(s_plan);
        const int n4 = (2 + g.plan[(size_t)ng * g.group_ints]) * (R / 4);   // header + records + sentinel
        for (int i = tid; i < n4; i += C::NT) dst[i] = src[i];
        for (int i = tid; i < C::FLAG_BYTES / 4; i += C::NT) s_done[i] = 0;
    }
    __syncthreads();
    const int ns = __builtin_amdgcn_readfirstlane(s_plan[0]);   // steps (k-pairs) per tile
    const int ne = __builtin_amdgcn_readfirstlane(s_plan[1]);   // entries per tile
    const int nsteps = ns * ntiles;                              // global steps of this workgroup

    // lane l: int l of the record of step s of a tile
    auto fetch_rec = [&](int s) -> int { return s_plan[(1 + s) * R + lane]; };

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
        // per token tile: global offsets of this wave's panel rows (rows past the end re-read the last
        // row; they are never stored)
        unsigned a_voff[C::A_PER_WAVE];
        const unsigned char* a_tile = A;
        auto enter_tile = [&](int j) {
            const int m0 = (p + j * g.wg_per_group) * C::BM;
            const int last_row = g.M - 1 - m0;
#pragma unroll
            for (int q = 0; q < C::A_PER_WAVE; ++q) {
                const int r = a_row[q] < last_row ? a_row[q] : last_row;
                a_voff[q] = (unsigned)r * (unsigned)a_row_bytes + a_chunk[q];
            }
            a_tile = uniform_ptr(A + (size_t)m0 * a_row_bytes);
        };
        // Issue the DMA of global step t (panel buffer `stage`, records in vrec, e0 entries before it).
        // The blocks of a step are dealt to the copy waves by entry number (dw, dw + 4, ...).
        // Returns the instruction count.
        auto issue_step = [&](unsigned stage, int vrec, int e0, int cnt) -> int {
            int n = 0;
            const int pair = __builtin_amdgcn_readlane(vrec, D16_F_PAIR);
            const unsigned char* src = uniform_ptr(a_tile + (size_t)pair * C::ROWB);
#pragma unroll
            for (int q = 0; q < C::A_PER_WAVE; ++q) dma16(stage + q * 1024, src, a_voff[q]);
            n = C::A_PER_WAVE;
#pragma unroll
            for (int k = 0; k < 2 * D16_NB / NP; ++k) {
                const int i = dw + k * NP;
                if (i < cnt) {
                    const unsigned id = (unsigned)__builtin_amdgcn_readlane(vrec, i);
                    const unsigned char* bsrc = uniform_ptr(D + ((size_t)id << 11));
                    const unsigned bdst = lds_b + (((unsigned)(e0 + i) & (RB - 1)) << 11);
                    dma16(bdst, bsrc, b_voff[0]);
                    dma16(bdst + 1024, bsrc, b_voff[1]);
                    n += 2;
                }
            }
            return n;
        };

        // minimum over the compute waves of (steps done, entries done): lanes 0..7 read lane 0's pair of
        // each wave, three row shifts bring the minimum to lane 7
        auto consumers_done = [&](int& steps, int& entries) {
            // every lane of a compute wave writes its own copy; reading copy w of wave w puts the 8 words on 8 banks
            const int* pw = s_done + (lane & 7) * 64 + (lane & 7);
            int a = lds_peek(pw), b = lds_peek(pw + NW * 64);
#define PBS_MIN_SHR(SH)                                                                  \
    {                                                                                    \
        const int a2 = __builtin_amdgcn_update_dpp(a, a, 0x110 + SH, 0xf, 0xf, false);   \
        const int b2 = __builtin_amdgcn_update_dpp(b, b, 0x110 + SH, 0xf, 0xf, false);   \
        a = a2 < a ? a2 : a;                                                             \
        b = b2 < b ? b2 : b;                                                             \
    }
            PBS_MIN_SHR(1) PBS_MIN_SHR(2) PBS_MIN_SHR(4)
#undef PBS_MIN_SHR
            steps = __builtin_amdgcn_readlane(a, 7);
            entries = __builtin_amdgcn_readlane(b, 7);
        };
        const unsigned landed_lds = (unsigned)(uintptr_t)(s_landed + dw * 64);
        int jn = 0, sn = 0;          // step t is step sn of tile jn
        int vrec = fetch_rec(0);
        unsigned stage = lds_a + dw * (C::A_PER_WAVE * 1024);   // this wave's part of panel buffer t % RS
        const unsigned stage_end = stage + RS * C::PANEL_BYTES;
        enter_tile(0);
        for (int t = 0; t < nsteps; ++t) {
            // wait until the panel buffer and the block slots of step t are free
            const int cnt = __popc((unsigned)__builtin_amdgcn_readlane(vrec, D16_F_MASK));
            const int e0 = jn * ne + __builtin_amdgcn_readlane(vrec, D16_F_CUM);
            const int end_t = e0 + cnt;
            bool free_now = false;
            for (int spin = 0; spin < C::SPIN_LIMIT; ++spin) {
                int steps, entries;
                consumers_done(steps, entries);
                if (steps >= t - RS + 1 && end_t - entries <= RB) {
                    free_now = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(D16_SLEEP);
            }
            // Cannot happen unless the protocol is broken: say so; the compute waves mark their results.
            if (!free_now) {
                lds_poke(s_fail, 1);
                count_protocol_failure();
            }
            wait_dma(63 - C::MAX_STEP_DMA - 1);   // the counter of outstanding loads has 6 bits
            asm volatile("" ::: "memory");
            const int n_t = issue_step(stage, vrec, e0, cnt);
            stage += C::PANEL_BYTES;
            if (stage == stage_end) stage -= RS * C::PANEL_BYTES;
            if (++sn == ns) {
                sn = 0;
                ++jn;
                if (t + 1 < nsteps) enter_tile(jn);
            }
            vrec = fetch_rec(sn);   // consumed in the next iteration: the LDS latency is hidden
#ifdef PBS_DDS16_PUBLISH_AFTER_WAIT
            // Checking build (libpbs_hip_check.so): the conservative protocol.  The copy wave waits until all its
            // loads have returned and only then writes the step number itself, so nothing depends on the order in
            // which one wave's LDS-DMA loads land.  Slower; its results must equal the product build's bit for bit.
            wait_dma(0);
            lds_poke(s_landed + dw * 64 + lane, (t + 1) & 255);
#else
            // behind the operands of step t: the number t + 1 (mod 256) onto this wave's landed words
            dma4(landed_lds, uniform_ptr(reinterpret_cast<const unsigned char*>(g.seq + ((t + 1) & 255))), 0u);
#endif
            (void)n_t;
        }
        wait_dma(0);
        return;
    }

    // =====================================================================================
    // compute waves
    // =====================================================================================
    const int ms = wave % C::NSL;       // token slice (TM * 32 tokens)
    const int quarter = wave / C::NSL;  // group of NBW block columns
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
    // fragments of one 16-byte register index q: 8 of the 16 k values a lane holds of a k-block
    auto load_a = [&](uint4 (&fa)[TM], const unsigned char* panel, int kk, int q) {
        const unsigned char* pq = panel + (a_lane_off ^ (kk * 64 + q * 16));
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const uint4*>(pq + i * 32 * C::ROWB);
    };
    auto load_b = [&](const unsigned char* pb, int q) -> uint4 {
        if constexpr (TRANS) {
            return *reinterpret_cast<const uint4*>(pb + (b_lane_off ^ (q * 16)));
        } else {
            const unsigned char* pp = pb + b_lane_off;
            const uint2 lo = tr16_b64(pp + (8 * q) * 64);
            const uint2 hi = tr16_b64(pp + (8 * q + 4) * 64);
            return make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
    };

    bf16_t* out = static_cast<bf16_t*>(g.out);
    const bf16_t* bias = static_cast<const bf16_t*>(g.bias);
    const int col0 = (nb0 + quarter * NBW) * 32;   // first result column of this wave
    bf16_t* stage = reinterpret_cast<bf16_t*>(smem + C::A_RING_BYTES + C::B_RING_BYTES + wave * C::STAGE_WAVE_BYTES);

    bool gave_up = false;   // a wait ran into its bound (broken protocol): results are marked NaN
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
        const bool failed = __builtin_amdgcn_readfirstlane(lds_peek(s_fail)) != 0;
        constexpr int CW = NBW < 4 ? NBW : 4;          // block columns staged at a time
        constexpr int CHUNKS = CW * 4;                 // 16-byte pieces per staged row
        constexpr int ROWS_PER_READ = 64 / CHUNKS;     // staged rows one wave-wide read covers
        bf16_t* st_w = stage + (4 * eh) * C::STAGE_ROW + er;                    // + vv rows, + jc*32
        const int rd_r = l / CHUNKS, rd_c = (l % CHUNKS) * 8;
        const bf16_t* st_r = stage + rd_r * C::STAGE_ROW + rd_c;                // + ROWS_PER_READ rows per further read
#pragma unroll
        for (int cg = 0; cg < NBW / CW; ++cg) {   // CW block columns at a time
            float bv[CW];
            {
                bf16_t braw[CW];   // all loads first: one wait
#pragma unroll
                for (int jc = 0; jc < CW; ++jc) {
                    const int col = col0 + (cg * CW + jc) * 32 + er;
                    braw[jc].bits = 0;
                    if (bias) braw[jc] = bias[col < g.N ? col : 0];
                }
#pragma unroll
                for (int jc = 0; jc < CW; ++jc) {
                    const int col = col0 + (cg * CW + jc) * 32 + er;
                    bv[jc] = col < g.N ? E::to_f32(braw[jc]) : 0.f;
                    if (gave_up || failed) bv[jc] = __builtin_nanf("");
                }
            }
            const int col = col0 + cg * CW * 32 + rd_c;
#pragma unroll
            for (int t = 0; t < TM; ++t) {
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
#pragma unroll
                    for (int jc = 0; jc < CW; ++jc)
#pragma unroll
                        for (int vv = 0; vv < 4; ++vv)
                            st_w[vv * C::STAGE_ROW + jc * 32] = E::from_f32(acc[t][cg * CW + jc][4 * gq + vv] + bv[jc]);
                    // both reads first: one wait for the staged rows instead of one per store
                    uint4 val[8 / ROWS_PER_READ];
#pragma unroll
                    for (int pp = 0; pp < 8 / ROWS_PER_READ; ++pp)
                        val[pp] = *reinterpret_cast<const uint4*>(st_r + pp * ROWS_PER_READ * C::STAGE_ROW);
#pragma unroll
                    for (int pp = 0; pp < 8 / ROWS_PER_READ; ++pp) {
                        const int row = m0 + (ms * TM + t) * 32 + gq * 8 + pp * ROWS_PER_READ + rd_r;
                        if (row < g.M && col < g.N) *reinterpret_cast<uint4*>(out + (size_t)row * g.N + col) = val[pp];
                    }
                }
            }
        }
    };

    // steps whose operands have arrived from every copy wave
    // Steps whose operands have arrived from every copy wave.  The words hold the count modulo 256 and
    // are never more than the ring depth away from u, so the signed 8-bit difference is exact.
    auto producers_landed = [&](int u) -> int {
        const int v = lds_peek(s_landed + (lane & 3) * 64 + (lane & 3));   // copy c of wave c: 4 banks
        int m = 127;
#pragma unroll
        for (int c = 0; c < NP; ++c) {
            const int d = (int)(signed char)(__builtin_amdgcn_readlane(v, c) - u);
            m = d < m ? d : m;
        }
        return u + m;
    };
    if (ns > 0) {
        int j = 0, s = 0;
        int landed = 0;
        int vrec = fetch_rec(0);
        for (int u = 0; u < nsteps; ++u) {
            if (landed <= u) {
                for (int spin = 0; spin < C::SPIN_LIMIT; ++spin) {
                    landed = producers_landed(u);
                    if (landed > u) break;
                    __builtin_amdgcn_s_sleep(D16_SLEEP);
                }
                // Operands that never arrive mean a broken protocol, not a slow machine (a wave that is
                // not running does not count polls).  Make the failure visible: the tiles become NaN.
                if (landed <= u) {
                    gave_up = true;
                    count_protocol_failure();
                }
            }
            asm volatile("" ::: "memory");   // operand reads stay behind the poll
            const unsigned mask = (unsigned)__builtin_amdgcn_readlane(vrec, D16_F_MASK);
            const int base = j * ne + __builtin_amdgcn_readlane(vrec, D16_F_CUM);
            const unsigned char* panel = a_ring + (u % RS) * C::PANEL_BYTES;
            if (++s == ns) s = 0;
            vrec = fetch_rec(s);   // the next step's record, needed after this step's products
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const unsigned mk = (mask >> (16 * kk)) & 0xffffu;
                const unsigned mine = (mk >> (NBW * quarter)) & ((1u << NBW) - 1u);
                if (mine == 0) continue;
                const int e0 = base + (kk ? __popc(mask & 0xffffu) : 0) + __popc(mk & ((1u << (NBW * quarter)) - 1u));
                // The panel fragments of the k-block (both register indices) stay in registers while its
                // blocks pass by; a block's two fragments are fetched together and feed four products, so
                // one LDS round trip is paid per 128 matrix-core cycles (the other wave of the SIMD fills
                // them).  The accumulator index stays static; the branches are wave-uniform.
                {
                    uint4 fa[2][TM];
                    load_a(fa[0], panel, kk, 0);
                    load_a(fa[1], panel, kk, 1);
                    int e = e0;
#pragma unroll
                    for (int jc = 0; jc < NBW; ++jc) {
                        if ((mine >> jc) & 1u) {
                            const unsigned char* pb = b_ring + (e & (RB - 1)) * C::BLK_BYTES;
                            const uint4 fb0 = load_b(pb, 0);
                            const uint4 fb1 = load_b(pb, 1);
                            ++e;
#pragma unroll
                            for (int t = 0; t < TM; ++t)
                                acc[t][jc] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                    __builtin_bit_cast(bf16x8, fa[0][t]), __builtin_bit_cast(bf16x8, fb0), acc[t][jc], 0, 0, 0);
#pragma unroll
                            for (int t = 0; t < TM; ++t)
                                acc[t][jc] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                    __builtin_bit_cast(bf16x8, fa[1][t]), __builtin_bit_cast(bf16x8, fb1), acc[t][jc], 0, 0, 0);
                        }
                    }
                }
            }
            // this wave has read everything it needs of step u: publish (steps, entries) done.  LDS
            // serves a wave's requests in order, so the reads above precede this write.
            asm volatile("" ::: "memory");
            {
                int* pd = s_done + wave * 64 + lane;   // same per-lane offset as the record reads
                lds_poke(pd, u + 1);
                lds_poke(pd + NW * 64, base + __popc(mask));
            }
            if (s == 0) {
                epilogue(j);
                zero_acc();
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
