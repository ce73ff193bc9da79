// dense x block-sparse -> dense for bf16, one block column per wave (forward and input gradient).
//
// Tile: 128 tokens x 16 block columns, owned by one workgroup of 16 waves (4 per SIMD).  Wave w owns one
// block column of the tile for all 128 tokens: four 32 x 32 accumulators with fixed register names.
// Its work is a list of items, one per stored block of its column, sorted by k; which accumulator a
// product goes to never depends on the pattern, so the loop over items is straight-line code: 8 loads of
// dense-operand fragments from LDS, 8 matrix instructions.
//
// What bounds this kernel is instruction issue: a SIMD issues at most one scalar, one vector, one LDS and one
// vector-memory instruction per four cycles, shared by its four waves, so every bookkeeping instruction of an
// item is paid several times over on the path of the wave with the most items.  Hence: everything that
// depends on the pattern only is precomputed in the item words; a wave looks at one progress word per item;
// waves that wait sleep long; and only a wave that has to wait anyway copies.
//
// The block columns are ranked by block count and dealt to the waves so that every SIMD of every
// workgroup gets the same number of blocks (ddsc_cols_kernel): places 0-3 of a group (one per SIMD) hold
// its heaviest columns, places 12-15 its lightest.  Adjacent block columns stay in one group, so that the
// two halves of a 128-byte line of the result are stored at about the same time.
//
// Operands.
//   dense operand   A step is a pair of adjacent k-blocks (128-byte rows).  Its 128 x 64 panel goes
//                   global -> LDS by DMA into a ring of RS steps (16 KB each).  A step is copied by
//                   whichever wave finds itself waiting for a panel while the step's ring slot is free
//                   (16 DMA instructions); up to RS copies are in flight at a time.
//   packed blocks   never pass through LDS.  A block is multiplied by exactly one wave per token tile, so
//                   the wave loads its two 16-byte fragments per lane straight from global memory into
//                   registers, DC_L items ahead, with ordinary loads (the compiler places the waits and never
//                   moves a register a load in flight is going to write).  That needs the block stored with
//                   k along its rows ([n][k]); the stored layout is that for the input gradient, the forward
//                   product is given a copy of the data with every block transposed (transpose_blocks_kernel),
//                   which, being a copy anyway, is written in the order the fragments are loaded in.
//   The LDS so freed makes the panel ring 8 steps deep.
//
// The product is computed transposed, acc[n][token] (block fragment as first operand): a lane then holds
// 4 consecutive result columns of one token per accumulator register quad; the two lane halves exchange
// quads (v_permlane32_swap) so that every lane stores 16 contiguous bytes of a result row, straight from
// the registers.
//
// Progress words in LDS (one writer each, only growing; no barriers after the prologue):
//   landed[s]   ring slot s holds step landed[s] - 1: behind the rows of step t the copying wave issues one
//               single-lane 4-byte DMA that copies the number t + 1 from a table 0, 1, 2, ... in global memory
//               onto the word of slot t % RS; a wave's loads complete in order;
//   done[w]     the global step wave w still needs: it has finished reading every earlier step (every lane
//               writes its own copy of the word, lane 0's is read);
//   next        the first step nobody has copied yet (advanced by compare-and-swap: the one word with several
//               writers).
// Step t may overwrite ring slot t % RS once min done[] > t - RS; an item of step u may be read when its
// slot's word exceeds u.  A wave reads that word for its next item behind the current item's fragment reads
// and looks at it when it gets there, so the round trip is off the item's path.  A wave whose panel is not
// there reads all the words at once, copies every free step it manages to claim, sleeps, and looks again:
// the waves with few items run ahead, meet steps that are not there yet and so do most of the copying, and a
// freed ring slot is refilled within one poll interval, whatever the other waves are busy with.  (With a
// fixed copier per step, a slot waited for that wave to finish its own item or its epilogue: 0.203 -> 0.186 ms
// for the input gradient of the 4096 x 4096 layer at density 0.25, 0.297 -> 0.274 at 0.5.)
// Every wait polls with s_sleep and is bounded; a wait that runs into its bound (a broken protocol, not a slow
// machine) makes the results NaN instead of passing silently.
//
// The compiler does not see the DMA instructions (inline assembly), so after a wave has copied, its next
// wait for a block also covers the DMA instructions issued since the block was requested: it waits for its
// own copy to land.  A wave that has not copied waits exactly.
//
// Persistent workgroups: a workgroup keeps one group of 16 block columns and walks several token
// tiles; steps are numbered across tiles, so the first loads of a tile overlap the previous tile's stores.
//
// Plan per group of 16 block columns (ddsc_plan_kernel), ints:
//   [0] ns = k-pairs any column touches   [1 + c] items of column c   [17] 1 if the lists are usable
//   [32 + c] block column of the result in place c (or -1)
//   [64 + s]                          k-pair index of step s
//   [64 + KP + 2 (c KB + i)]          item i of column c: step | (k & 1) << 9 | (1 << 10 if it is the column's last)
//   [64 + KP + 2 (c KB + i) + 1]      byte offset in the data of the block of the column's item i + DC_L (cyclically)
//   (KP = K / 64, KB = K / 32)
#pragma once
#include <type_traits>

#include "pbs_common.h"

namespace pbs {

constexpr int DC_NB = 16;               // block columns per tile = waves per workgroup
constexpr int DC_NC = 8;                // words reserved for landed[] (one per ring slot)
constexpr int DC_L = 2;                 // blocks loaded ahead of the item being multiplied
constexpr int DC_BM = 128;              // tokens per tile
constexpr int DC_HDR = 64;
constexpr int DC_H_COL = 32;
constexpr int DC_MAX_KP = 512;          // k-pairs (K <= 32768): 9 bits of an item
constexpr int DC_ITEM_LAST = 1 << 10;
constexpr int DC_MAX_BLOCKS = 1 << 21;  // byte offsets of blocks stay below 2^32
constexpr int DC_ITEMS_LDS = 2048;      // items of a group kept in LDS (every pattern up to K = 4096)
constexpr int DC_SEQ_INTS = 16384;      // the table 0, 1, 2, ...: a workgroup's steps are numbered below this (a power of two)
#ifndef DC_SLEEP
#define DC_SLEEP 8
#endif
static inline size_t ddsc_plan_group_ints(int KB) { return (size_t)DC_HDR + (KB / 2) + (size_t)DC_NB * 2 * KB; }

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// Which block column sits in which place of which group: cols[16 g + c], or -1.  Natural order unless the
// per-column block counts differ; then the columns are ranked by count and dealt in serpentine order to
// the SIMD quarters of the groups (place c runs on SIMD c % 4), so that every SIMD of every workgroup gets
// about the same number of blocks.  One workgroup.
constexpr int DC_BALANCE_MAX_COLS = 4096;
__global__ __launch_bounds__(256) void ddsc_cols_kernel(const int32_t* __restrict__ ptr, int nblk_n, int n_groups, int nnz,
                                                        int* cols) {
    constexpr int NT = 256;
    __shared__ int s_cnt[DC_BALANCE_MAX_COLS];
    const int tid = threadIdx.x;
    const int total = n_groups * DC_NB;
    if (nblk_n > DC_BALANCE_MAX_COLS) {
        for (int i = tid; i < total; i += NT) cols[i] = i < nblk_n ? i : -1;
        return;
    }
    for (int i = tid; i < total; i += NT) cols[i] = -1;
    for (int c = tid; c < nblk_n; c += NT) s_cnt[c] = clamp_entry(ptr[c + 1], nnz) - clamp_entry(ptr[c], nnz);
    __syncthreads();
    // Adjacent columns 2 q, 2 q + 1 stay together (places s and s + 4 of one group): their waves store the two halves
    // of the same 128-byte lines of the result at about the same time, so the lines reach memory whole.
    const int units = 4 * n_groups;   // SIMD quarters: 4 places = 2 pairs each
    const int npairs = (nblk_n + 1) / 2;
    for (int q = tid; q < npairs; q += NT) {
        const int c0 = 2 * q, c1 = 2 * q + 1;
        const int n = s_cnt[c0] + (c1 < nblk_n ? s_cnt[c1] : 0);
        int rank = 0;
        for (int o = 0; o < npairs; ++o) {
            const int m = s_cnt[2 * o] + (2 * o + 1 < nblk_n ? s_cnt[2 * o + 1] : 0);
            rank += (m > n || (m == n && o < q)) ? 1 : 0;
        }
        const int turn = rank / units;             // 0 or 1: which of the quarter's 2 pairs
        int u = rank % units;
        if (turn & 1) u = units - 1 - u;           // serpentine: heavy and light pairs share a quarter
        // quarter u = (group u / 4, SIMD u % 4); the pair's places are SIMD + 8 * turn and 4 more
        const int place = (u >> 2) * DC_NB + (u & 3) + 8 * turn;
        cols[place] = c0;
        if (c1 < nblk_n) cols[place + 4] = c1;
    }
}

// One workgroup per group of 16 block columns.
__global__ __launch_bounds__(256) void ddsc_plan_kernel(const int32_t* __restrict__ ptr, const int32_t* __restrict__ idx,
                                                        const int* __restrict__ cols, int nblk_n, int KB, int nnz, int* plan,
                                                        int group_ints, int* seq) {
    __shared__ int s_rank[DC_MAX_KP + 1];
    __shared__ int s_lo[DC_NB], s_hi[DC_NB];
    __shared__ int s_part[256];
    const int tid = threadIdx.x;
    const int KP = KB / 2;
    int* out = plan + (size_t)blockIdx.x * group_ints;
    if (tid < DC_NB) {
        const int c = cols[blockIdx.x * DC_NB + tid];
        const bool ok = c >= 0 && c < nblk_n;
        s_lo[tid] = ok ? clamp_entry(ptr[c], nnz) : 0;
        s_hi[tid] = ok ? clamp_entry(ptr[c + 1], nnz) : 0;
        out[DC_H_COL + tid] = ok ? c : -1;
    }
    for (int i = tid; i <= KP; i += 256) s_rank[i] = 0;
    __syncthreads();
    // k-pairs present
    for (int c = 0; c < DC_NB; ++c)
        for (int e = s_lo[c] + tid; e < s_hi[c]; e += 256) {
            const int kb = idx[2 * e], b = idx[2 * e + 1];
            if (kb >= 0 && kb < KB && b >= 0 && b < nnz) s_rank[kb >> 1] = 1;
        }
    __syncthreads();
    // exclusive prefix sum over the k-pairs (KP <= 512: two per thread, then a scan over 256 partial sums)
    const int p0 = 2 * tid, p1 = 2 * tid + 1;
    const int f0 = p0 < KP ? s_rank[p0] : 0, f1 = p1 < KP ? s_rank[p1] : 0;
    s_part[tid] = f0 + f1;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
        const int v = tid >= d ? s_part[tid - d] : 0;
        __syncthreads();
        s_part[tid] += v;
        __syncthreads();
    }
    const int before = s_part[tid] - (f0 + f1);
    const int ns = s_part[255];
    if (p0 < KP) {
        s_rank[p0] = before;
        if (f0) out[DC_HDR + before] = p0;
    }
    if (p1 < KP) {
        s_rank[p1] = before + f0;
        if (f1) out[DC_HDR + before + f0] = p1;
    }
    __syncthreads();
    // items: thread c walks column c's entries (sorted by k; entries that are not are dropped)
    if (tid < DC_NB) {
        int* items = out + DC_HDR + KP + (size_t)tid * 2 * KB;
        int n = 0, last = -1;
        for (int e = s_lo[tid]; e < s_hi[tid]; ++e) {
            const int kb = idx[2 * e], b = idx[2 * e + 1];
            if (kb > last && kb < KB && b >= 0 && b < nnz && b < DC_MAX_BLOCKS) {
                items[2 * n] = s_rank[kb >> 1] | ((kb & 1) << 9);
                items[2 * n + 1] = b;   // for now: the item's own block
                ++n;
                last = kb;
            }
        }
        if (n > 0) items[2 * (n - 1)] |= DC_ITEM_LAST;
        out[1 + tid] = n;
    }
    if (tid == 0) {
        out[0] = ns;
        out[17] = 1;
    }
    if (tid >= 18 && tid < DC_H_COL) out[tid] = 0;
    if (tid >= DC_H_COL + DC_NB && tid < DC_HDR) out[tid] = 0;
    // the numbers the waves publish their copies with
    for (int i = blockIdx.x * 256 + tid; i < DC_SEQ_INTS; i += gridDim.x * 256) seq[i] = i;
}
// Second pass over the plan: the second word of item i becomes the byte offset of the block of item i + DC_L (cyclically).
// One workgroup per group; thread c does column c (in place: the rotation is done through a few registers).
__global__ __launch_bounds__(64) void ddsc_plan_ahead_kernel(int KB, int* plan, int group_ints) {
    const int tid = threadIdx.x;
    if (tid >= DC_NB) return;
    int* out = plan + (size_t)blockIdx.x * group_ints;
    const int KP = KB / 2;
    const int n = out[1 + tid];
    if (n <= 0) return;
    int* items = out + DC_HDR + KP + (size_t)tid * 2 * KB;
    // the first DC_L blocks are needed again at the end
    int first[DC_L];
#pragma unroll
    for (int i = 0; i < DC_L; ++i) first[i] = items[2 * (i % n) + 1];
    for (int i = 0; i < n; ++i) {
        const int src = i + DC_L;
        int b;
        if (src < n) b = items[2 * src + 1];
        else {
            const int r = (src - n) % n;   // wrapped: one of the first blocks (n may be smaller than DC_L)
            b = r < DC_L ? first[r] : items[2 * r + 1];
        }
        items[2 * i + 1] = (int)((unsigned)b << 11);
    }
}

// data_t block b = data block b (stored [k][n], 32 x 32 elements of 2 bytes) in the order ddsc_kernel<RS, true> loads it:
// [half q of k][lane = 32 h + n][8 k values], k = 16 q + 8 h + e, so that a wave's load of one fragment is 1 KB of
// consecutive bytes (8 whole cache lines instead of half of each of the block's 16).  One wave per block.
__global__ __launch_bounds__(256) void transpose_blocks_kernel(const uint16_t* __restrict__ data, uint16_t* __restrict__ data_t,
                                                               int nnz) {
    __shared__ uint16_t s[4][32][34];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int b = blockIdx.x * 4 + w;
    if (b >= nnz) return;
    const uint16_t* src = data + (size_t)b * 1024;
    uint16_t* dst = data_t + (size_t)b * 1024;
    // lane l reads 16 elements: row l / 2, columns 16 (l % 2) .. + 15
    const int r = lane >> 1, c0 = (lane & 1) * 16;
    const uint4 v0 = *reinterpret_cast<const uint4*>(src + r * 32 + c0);
    const uint4 v1 = *reinterpret_cast<const uint4*>(src + r * 32 + c0 + 8);
    const uint32_t wv[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        s[w][c0 + 2 * i][r] = (uint16_t)(wv[i] & 0xffffu);
        s[w][c0 + 2 * i + 1][r] = (uint16_t)(wv[i] >> 16);
    }
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    uint32_t o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (uint32_t)s[w][r][c0 + 2 * i] | ((uint32_t)s[w][r][c0 + 2 * i + 1] << 16);
    // this lane holds k = 16 q .. 16 q + 15 of result column n = r, with q = lane % 2
    const int q = lane & 1;
    *reinterpret_cast<uint4*>(dst + q * 512 + r * 8) = make_uint4(o[0], o[1], o[2], o[3]);          // h = 0
    *reinterpret_cast<uint4*>(dst + q * 512 + (32 + r) * 8) = make_uint4(o[4], o[5], o[6], o[7]);   // h = 1
}



struct DdscArgs {
    const void* a;         // [M, K] row-major bf16
    const void* data;      // [nnz*32, 32] bf16, every block stored [n][k] (FM = false) or in fragment order (FM = true)
    const int* plan;       // built by ddsc_plan_kernel + ddsc_plan_ahead_kernel for this pattern and direction
    const int* seq;        // the table 0, 1, 2, ... written by ddsc_plan_kernel
    const void* bias;      // nullptr or [N]
    void* out;             // [M, N] row-major
    int M, N, K, nnz;
    int m_tiles, n_groups, group_ints;
    int wg_per_group;      // workgroups that share the token tiles of one column group
};

template <int RS>
struct DdscCfg {
    static constexpr int NW = DC_NB, NT = NW * 64, BM = DC_BM;
    static constexpr int ROWB = 128;                   // one panel row: 64 k values
    static constexpr int PANEL_BYTES = BM * ROWB;      // 16 KB per step
    static constexpr int A_RING_BYTES = RS * PANEL_BYTES;
    static constexpr int ITEMS_OFF = A_RING_BYTES;                       // two words per item
    static constexpr int STEPS_OFF = ITEMS_OFF + DC_ITEMS_LDS * 8;
    static constexpr int DONE_OFF = STEPS_OFF + DC_MAX_KP * 4;           // done[16][64]
    static constexpr int LANDED_OFF = DONE_OFF + NW * 256;               // landed[8], failure word
    static constexpr int BIAS_OFF = LANDED_OFF + 256;                    // bias[16][32], 2 bytes each
    static constexpr int LDS_BYTES = BIAS_OFF + NW * 64;
    static constexpr int SPIN_LIMIT = 1 << 18;
    static_assert(RS >= 4 && RS <= 8, "ring depth");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

// 4-byte DMA with only lane 0 active: the word at base to the LDS word at lds_base
static __device__ __forceinline__ void dma4_lane0(unsigned lds_base_uniform, const unsigned char* base_uniform) {
    uint64_t saved;
    lds_base_uniform = __builtin_amdgcn_readfirstlane(lds_base_uniform);
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 1\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3\n\ts_mov_b64 exec, %0\n\t"
                 : "=&s"(saved)
                 : "s"(lds_base_uniform), "v"(0u), "s"(base_uniform)
                 : "memory");
}

template <int RS, bool FM>
__global__ __launch_bounds__(DC_NB * 64) void ddsc_kernel(DdscArgs g) {
    static_assert(RS <= DC_NC, "one landed word per ring slot");
    using C = DdscCfg<RS>;
    using E = Elem<bf16_t>;
    constexpr int NW = C::NW, NC = DC_NC, L = DC_L;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    unsigned char* const a_ring = smem;
    int* const s_items = reinterpret_cast<int*>(smem + C::ITEMS_OFF);
    int* const s_steps = reinterpret_cast<int*>(smem + C::STEPS_OFF);
    int* const s_done = reinterpret_cast<int*>(smem + C::DONE_OFF);       // [16][64]
    int* const s_landed = reinterpret_cast<int*>(smem + C::LANDED_OFF);   // [8]
    int* const s_fail = s_landed + NC;
    const unsigned lds_a = (unsigned)(uintptr_t)a_ring;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Workgroup -> (column group, first token tile).  The workgroups of one XCD (blockIdx % 8) cover half of the
    // column groups and every fourth token stream (with an odd number of groups: all groups, every eighth stream),
    // so a panel is fetched into two L2s and the blocks an XCD keeps re-reading (once per token tile) are 4 MB
    // at 4096 x 4096, which its L2 holds.  All groups per XCD (a panel in one L2, 8 MB of blocks) is 1.2 % slower
    // at both densities, a quarter of the groups per XCD 6 % slower at density 0.25.
    const int wg = blockIdx.x;
    int ng, p;
    if ((g.n_groups & 1) == 0) {
        const int x = wg & 7, r = wg >> 3, gs = g.n_groups >> 1;
        ng = (x & 1) * gs + (r % gs);
        p = (x >> 1) + 4 * (r / gs);
    } else {
        ng = (wg >> 3) % g.n_groups;
        p = (wg & 7) + 8 * ((wg >> 3) / g.n_groups);
    }
    if (p >= g.wg_per_group) return;
    const int ntiles = (g.m_tiles - p + g.wg_per_group - 1) / g.wg_per_group;   // token tiles p, p + P, ...

    const int KB = g.K / 32, KP = KB / 2;
    const int* gplan = g.plan + (size_t)ng * g.group_ints;
    // the header, one int per lane
    const int v_hdr = gplan[lane];
    const int ns = __builtin_amdgcn_readlane(v_hdr, 0);
    const int my_col = __builtin_amdgcn_readlane(v_hdr, DC_H_COL + wave);
    const bool has_col = my_col >= 0 && my_col * 32 < g.N;
    const int ni = has_col ? __builtin_amdgcn_readlane(v_hdr, 1 + wave) : 0;
    // items of the group -> LDS, column after column (the host launches this kernel only when they fit: K <= 4096)
    int ioff = 0;
    {
        int off = 0;
#pragma unroll
        for (int c = 0; c < NW; ++c) {
            const int n = __builtin_amdgcn_readlane(v_hdr, 1 + c);
            if (c == wave) ioff = off;
            if (off + n <= DC_ITEMS_LDS)
                for (int i = tid; i < 2 * n; i += C::NT) s_items[2 * off + i] = gplan[DC_HDR + KP + c * 2 * KB + i];
            off += n;
        }
        for (int i = tid; i < ns; i += C::NT) s_steps[i] = gplan[DC_HDR + i];
        for (int i = tid; i < NW * 64 + 64; i += C::NT) s_done[i] = 0;   // done, landed, failure word
        // the bias of this wave's 32 result columns (zeros without one): the stores of a tile must not wait for a load
        if (lane < 16) {
            uint32_t b2 = 0u;
            if (g.bias && has_col) b2 = reinterpret_cast<const uint32_t*>(static_cast<const bf16_t*>(g.bias) + my_col * 32)[lane];
            reinterpret_cast<uint32_t*>(smem + C::BIAS_OFF)[wave * 16 + lane] = b2;
        }
    }
    __syncthreads();
    const int* const my_items = s_items + 2 * ioff;
    auto item_word = [&](int i, int w) __attribute__((always_inline)) -> int {   // word w of item i; every lane reads the same
        return __builtin_amdgcn_readfirstlane(my_items[2 * i + w]);
    };

    const int nsteps = ns * ntiles;   // global steps of this workgroup (the host keeps this below DC_SEQ_INTS)
    const unsigned char* A = static_cast<const unsigned char*>(g.a);
    const unsigned char* Dp = static_cast<const unsigned char*>(g.data);
    const unsigned a_row_bytes = (unsigned)g.K * 2u;

    // ---------------- copy side: a wave that waits, copies ----------------
    // s_next = the first step nobody has copied yet.  A wave that has to wait for a panel (or has no items left) reads all
    // progress words; while the ring slot of step s_next is free (every wave needs a later step than s_next - RS) it claims
    // that step with a compare-and-swap on s_next and copies it: 128 rows, then the step's number behind them.  The waves
    // with few items run ahead, meet steps that are not there yet and so do most of the copying; the waves with many items
    // only copy when everything has run dry.
    int* const s_next = s_fail + 1;
    // t / ns = (t * magic) >> 32 for the step numbers of a workgroup (below 2^16) and 2 <= ns <= 512
    const unsigned magic_ns = ns > 1 ? 0xFFFFFFFFu / (unsigned)ns + 1u : 0u;
    bool gave_up = false;
    int md = 0;            // last minimum of done[] seen (it only grows)

    // Lane l of DMA instruction i of a step: row 8 i + l / 8, physical chunk l % 8 = logical chunk (l % 8) ^ ((row / 2) % 8):
    // the swizzle term is (l / 16) for even i and (l / 16) ^ 4 for odd i, so two per-lane offsets serve all rows (the row
    // advances in the scalar base address).
    auto copy_step = [&](int t) __attribute__((always_inline)) {   // all rows of step t, then the number t + 1 behind them
        t = __builtin_amdgcn_readfirstlane(t);   // the same in every lane; the DMA helpers want their bases in scalar registers
        // (tile, step and k-pair are in range by construction; they are clamped all the same, because they make addresses)
        int tile_c = ns > 1 ? (int)__builtin_amdgcn_readfirstlane((int)__umulhi((unsigned)t, magic_ns)) : t;
        tile_c = tile_c < ntiles ? tile_c : ntiles - 1;
        int step_c = t - tile_c * ns;
        step_c = step_c < 0 ? 0 : (step_c >= ns ? ns - 1 : step_c);
        const int m0 = (p + tile_c * g.wg_per_group) * C::BM;
        const int a_last_row = g.M - 1 - m0;   // last valid row of the tile (rows past the end re-read it; they are never stored)
        int pair = __builtin_amdgcn_readfirstlane(s_steps[step_c]);
        pair = pair < 0 ? 0 : (pair >= KP ? KP - 1 : pair);
        const unsigned char* src = uniform_ptr(A + (size_t)m0 * a_row_bytes + (size_t)pair * C::ROWB);
        const unsigned stage = __builtin_amdgcn_readfirstlane(lds_a + ((unsigned)t % (unsigned)RS) * C::PANEL_BYTES);
        // (per-lane values are derived from the lane id behind an opaque copy: kept across the item loop they
        // would cost registers the accumulators and fragments need.  A rolled loop: this code must stay small.)
        int lc = lane;
        asm volatile("" : "+v"(lc));
        const unsigned voff_row = (unsigned)(lc >> 3) * a_row_bytes;
        const unsigned voff_even = voff_row + (unsigned)(((lc & 7) ^ (lc >> 4)) * 16);
        const unsigned voff_odd = voff_row + (unsigned)(((lc & 7) ^ (lc >> 4) ^ 4) * 16);
#pragma unroll 1
        for (int i = 0; i < C::BM / 8; i += 2) {
            if (8 * i + 15 <= a_last_row) {
                // all 16 rows exist
                const unsigned char* src_i = uniform_ptr(src + (size_t)(8 * i) * a_row_bytes);
                dma16(stage + i * 1024, src_i, voff_even);
                dma16(stage + i * 1024 + 1024, src_i, voff_odd + 8u * a_row_bytes);
            } else {
                // rows past the end of the matrix re-read its last row
                const int l = lc;
#pragma unroll
                for (int ii = 0; ii < 2; ++ii) {
                    const int row = 8 * (i + ii) + (l >> 3);
                    const int r = row < a_last_row ? row : a_last_row;   // row of the tile, never negative
                    const unsigned voff = (unsigned)r * a_row_bytes + (unsigned)(((l & 7) ^ ((row >> 1) & 7)) * 16);
                    dma16(stage + (i + ii) * 1024, src, voff);
                }
            }
        }
#ifdef PBS_DDSC_PUBLISH_AFTER_WAIT
        // checking build: wait for the rows, then write the number (relies on no ordering of one wave's loads)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (lane == 0) lds_poke(s_landed + (t & (RS - 1)), t + 1);
#else
        dma4_lane0((unsigned)(uintptr_t)(s_landed + (t & (RS - 1))),
                   uniform_ptr(reinterpret_cast<const unsigned char*>(g.seq + ((t + 1) & (DC_SEQ_INTS - 1)))));
#endif
    };

    // ---------------- progress words ----------------
    // The landed word of step u's ring slot (every lane reads the same word).
    auto poll_issue = [&](int u) __attribute__((always_inline)) -> int { return lds_peek(s_landed + (u & (RS - 1))); };
    auto poll_landed = [&](int v, int u) __attribute__((always_inline)) -> bool { return __builtin_amdgcn_readfirstlane(v) > u; };
    // All progress words in one read: lanes 0..15 done[lane], lane 16 the landed word of step u's slot, lane 17 s_next.
    auto poll_all = [&](int u) __attribute__((always_inline)) -> int {
        int l = lane;
        asm volatile("" : "+v"(l));
        // byte offsets from s_landed: done[l] lies NW * 256 bytes before it, s_next NC + 1 words behind it
        const int off = l < 16 ? l * 256 - NW * 256 : (l == 16 ? (u & (RS - 1)) * 4 : (NC + 1) * 4);
        return lds_peek(reinterpret_cast<const int*>(reinterpret_cast<const unsigned char*>(s_landed) + off));
    };
    // the minimum of done[] (-> md)
    auto poll_done = [&](int v) __attribute__((always_inline)) {
#define PBS_MIN_SHR(SH)                                                                \
    {                                                                                  \
        const int v2 = __builtin_amdgcn_update_dpp(v, v, 0x110 + SH, 0xf, 0xf, false); \
        v = v2 < v ? v2 : v;                                                           \
    }
        PBS_MIN_SHR(1) PBS_MIN_SHR(2) PBS_MIN_SHR(4) PBS_MIN_SHR(8)
#undef PBS_MIN_SHR
        const int dmin = __builtin_amdgcn_readlane(v, 15);
        md = dmin > md ? dmin : md;
    };
    auto publish_done = [&](int u) __attribute__((always_inline)) {
        int l = lane;
        asm volatile("" : "+v"(l));
        lds_poke(s_done + wave * 64 + l, u);
    };
    // Copy every step whose ring slot is free and that this wave manages to claim; v = the words poll_all has read.
    // Returns the value of s_next as far as this wave knows.
    auto copy_free_steps = [&](int v) __attribute__((always_inline)) -> int {
        int nc = __builtin_amdgcn_readlane(v, 17);
        poll_done(v);
        while (nc < nsteps && nc - RS < md) {
            int expected = nc;
            if (lane == 0)
                __hip_atomic_compare_exchange_strong((lds_int*)s_next, &expected, nc + 1, __ATOMIC_RELAXED,
                                                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            expected = __builtin_amdgcn_readfirstlane(expected);   // what s_next held: nc if the claim is this wave's
            if (expected == nc) {
                copy_step(nc);
                ++nc;
            } else {
                nc = expected;
            }
        }
        return nc;
    };
    // wait until step u has landed, copying what is free meanwhile
    auto slow_wait = [&](int u) __attribute__((always_inline)) {
        bool here = false;
        for (int spin = 0; spin < C::SPIN_LIMIT; ++spin) {
            const int v = poll_all(u);
            here = __builtin_amdgcn_readlane(v, 16) > u;
            if (here) break;
            copy_free_steps(v);
            // another wave has given up: so does this one
            if ((spin & 1023) == 1023 && __builtin_amdgcn_readfirstlane(lds_peek(s_fail)) != 0) break;
            __builtin_amdgcn_s_sleep(DC_SLEEP);
        }
        if (!here) {
            gave_up = true;
            if (lane == 0) lds_poke(s_fail, 1);
            count_protocol_failure();
        }
    };
    // after the last item: help until every step of the workgroup has been copied
    auto copy_rest = [&]() __attribute__((always_inline)) {
        for (int spin = 0; spin < C::SPIN_LIMIT && !gave_up; ++spin) {
            const int before = md;
            if (copy_free_steps(poll_all(0)) >= nsteps) break;
            if (md != before) spin = 0;
            if ((spin & 1023) == 1023 && __builtin_amdgcn_readfirstlane(lds_peek(s_fail)) != 0) break;
            __builtin_amdgcn_s_sleep(DC_SLEEP);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // ---------------- compute side ----------------
    const int lrow = lane & 31;
    const int h = lane >> 5;
    // dense-operand fragment q of token slice t, k-block kk of the panel in ring slot s: 16 bytes at
    //   16384 s + (32 t + lrow) * 128 + ((4 kk + 2 q + h) ^ swizzle(lrow)) * 16  =  (a_pre ^ (16384 s + 64 kk + 32 q)) + 4096 t
    const unsigned a_pre = (unsigned)(lrow * C::ROWB + ((h ^ ((lrow >> 1) & 7)) * 16));   // offset within a_ring
    static_assert((RS & (RS - 1)) == 0, "the ring slot is a bit field of the address");
    // block fragment q: row lrow of the [n][k] block, 16 bytes at 16 (2 q + h)
    // (or, in fragment order, 16 bytes at 1024 q + 16 lane)
    const unsigned b_lane = FM ? (unsigned)(lane * 16) : (unsigned)(lrow * 64 + h * 16);

    bf16_t* out = static_cast<bf16_t*>(g.out);

    f32x16 acc[4];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    };
    zero_acc();

    // Stores of one tile, straight from the accumulators.  Register quad q of a lane holds result columns
    // 8 q + 4 h .. + 3 of token (lane % 32) of a slice.  The lane halves swap quads so that the lower half holds
    // columns 8 q .. + 7 of quad q = 2 qq and the upper half those of quad q = 2 qq + 1: 16 contiguous bytes per lane.
    auto epilogue = [&](int j) __attribute__((always_inline)) {
        if (!has_col) return;
        const int m0 = (p + j * g.wg_per_group) * C::BM;
        const bool failed = gave_up || __builtin_amdgcn_readfirstlane(lds_peek(s_fail)) != 0;
        int l = lane;
        asm volatile("" : "+v"(l));
        const int r16 = l & 15, upper = (l >> 4) & 1, eh = l >> 5;
        // after the exchanges below a lane stores, per token slice, piece (upper, eh) = result columns 8 (2 upper + eh) .. + 7
        // of token r16 and of token 16 + r16: the four lanes of a token write 64 contiguous bytes in one instruction
        const int n0 = my_col * 32 + 8 * (2 * upper + eh);
        uint32_t bw[2][4];
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            const uint4 braw = *reinterpret_cast<const uint4*>(smem + C::BIAS_OFF + wave * 64 + 16 * (2 * qq + eh));
            bw[qq][0] = braw.x;
            bw[qq][1] = braw.y;
            bw[qq][2] = braw.z;
            bw[qq][3] = braw.w;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t w[2][4];   // piece qq of this lane's token (lane % 32): result columns 8 (2 qq + eh) .. + 7, as bf16 pairs
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                float x[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    // a = quad 2 qq (both halves), b = quad 2 qq + 1: after the swap a = [a lower, b lower], b = [a upper, b upper]
                    const unsigned a = __float_as_uint(acc[t][4 * (2 * qq) + e]);
                    const unsigned b = __float_as_uint(acc[t][4 * (2 * qq + 1) + e]);
                    const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
                    x[e] = __uint_as_float(r[0]);       // column 8 q' + e of this lane's quad q'
                    x[4 + e] = __uint_as_float(r[1]);   // column 8 q' + 4 + e
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float lo = x[2 * e] + __uint_as_float(bw[qq][e] << 16);
                    float hi = x[2 * e + 1] + __uint_as_float(bw[qq][e] & 0xffff0000u);
                    if (failed) lo = hi = __builtin_nanf("");
                    w[qq][e] = (uint32_t)E::from_f32(lo).bits | ((uint32_t)E::from_f32(hi).bits << 16);
                }
            }
            // The lanes 16..31 of each half hand their piece 0 to the lanes 0..15 and take those lanes' piece 1
            // (v_permlane16_swap: rows of 16 lanes; the odd rows of the first operand change places with the even rows of
            // the second).  Then every lane holds one piece of token r16 (first operand) and one of token 16 + r16 (second).
            uint32_t lo16[4], hi16[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const auto r = __builtin_amdgcn_permlane16_swap(w[0][e], w[1][e], false, false);
                lo16[e] = r[0];
                hi16[e] = r[1];
            }
            const int row = m0 + t * 32 + r16;
            // Non-temporal stores: the result (128 MiB at the benchmark shape) is not read again by this kernel, and
            // written the ordinary way it pushes the operands of the next product out of the last-level cache (the
            // weight gradient behind the input gradient 0.223 -> 0.207 ms, the whole step 0.589 -> 0.566).
            if (row < g.M) {
                const u32x4 vlo = {lo16[0], lo16[1], lo16[2], lo16[3]};
                __builtin_nontemporal_store(vlo, reinterpret_cast<u32x4*>(out + (size_t)row * g.N + n0));
            }
            if (row + 16 < g.M) {
                const u32x4 vhi = {hi16[0], hi16[1], hi16[2], hi16[3]};
                __builtin_nontemporal_store(vhi, reinterpret_cast<u32x4*>(out + (size_t)(row + 16) * g.N + n0));
            }
        }
    };

    if (ns == 0 || ni == 0) {
        // nothing to multiply in this column: the wave only helps copying; its result columns are the bias
        publish_done(0x7fffffff);
        for (int j = 0; j < ntiles; ++j) epilogue(j);
        if (ns > 0) copy_rest();
        return;
    }

    // Block fragments: L + 1 register sets, item i uses set i % (L + 1); the block of item i + L is loaded while
    // item i is worked on, into the set item i - 1 has just finished with.
    u32x4 fb[L + 1][2];
    auto load_block = [&](u32x4& b0, u32x4& b1, unsigned byte_off) __attribute__((always_inline)) {
        // plain loads: the compiler places the wait before their first use
        const unsigned char* pb = Dp + (size_t)(byte_off + b_lane);
        b0 = *reinterpret_cast<const u32x4*>(pb);
        b1 = *reinterpret_cast<const u32x4*>(pb + (FM ? 1024 : 32));
    };
    // the blocks of the first L items: item i's block offset is the second word of item i - L (cyclically)
#pragma unroll
    for (int i = 0; i < L; ++i) {
        int src = (i - L) % ni;
        if (src < 0) src += ni;
        load_block(fb[i][0], fb[i][1], (unsigned)item_word(src, 1));
    }
    // Items: 64 of them at a time sit in two registers (one per lane) and are picked with v_readlane; lists of more
    // than 64 items are read from memory item by item.
    const bool small = ni <= 64;
    const int li = lane < ni ? lane : 0;
    int vw0 = 0, vw1 = 0;
    if (small) {
        vw0 = my_items[2 * li];
        vw1 = my_items[2 * li + 1];
        asm volatile("" : "+v"(vw0), "+v"(vw1));
    }
    int idx = 0, j = 0;
    int item = small ? __builtin_amdgcn_readlane(vw0, 0) : item_word(0, 0);
    int u_base = 0;        // tile j's first global step
    int u = item & 511;
    publish_done(u);
    int raw = poll_issue(u);   // the progress words for the item a wave is about to start are read during the previous one


    // one item; S = the register set its block was loaded into; SMALL = the list is in registers
    auto do_item = [&](auto S_, auto SMALL_) __attribute__((always_inline)) {
        constexpr int S = decltype(S_)::value;
        constexpr bool SMALL = decltype(SMALL_)::value;
        constexpr int SF = (S + L) % (L + 1);
        // has this item's step landed?  (the read is always consumed: one left pending on one path costs a full wait at the join)
        const bool here = poll_landed(raw, u);
        if (!here && !gave_up) slow_wait(u);   // after a failed wait nothing is waited for any more: the results are void
        // the block of item idx + L, and the next item (behind the last item of the last tile: the list's first again)
        const bool last = (item & DC_ITEM_LAST) != 0;
        const int idx_n = last ? 0 : idx + 1;
        unsigned boff;
        int item_n;
        if constexpr (SMALL) {
            boff = (unsigned)__builtin_amdgcn_readlane(vw1, idx);
            item_n = __builtin_amdgcn_readlane(vw0, idx_n);
        } else {
            boff = (unsigned)item_word(idx, 1);
            item_n = item_word(idx_n, 0);
        }
        const int u_base_n = last ? u_base + ns : u_base;
        const int u_n = u_base_n + (item_n & 511);
        load_block(fb[SF][0], fb[SF][1], boff);
        __builtin_amdgcn_sched_barrier(0);
        // this item's dense-operand fragments, first half of k
        const unsigned sel = ((unsigned)(u & (RS - 1)) << 14) | (unsigned)((item >> 3) & 64);   // ring slot, k-block of the pair
        const unsigned ad0 = a_pre ^ sel, ad1 = ad0 ^ 32u;
        // (pointers derived from the LDS array itself: an integer turned into a pointer would be a flat address)
        const unsigned char* pa0 = a_ring + ad0;
        const unsigned char* pa1 = a_ring + ad1;
        uint4 a0[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) a0[t] = *reinterpret_cast<const uint4*>(pa0 + t * 4096);
        // the progress words for the next item, behind the fragment reads
        raw = poll_issue(u_n);
        const bf16x8 w0 = __builtin_bit_cast(bf16x8, fb[S][0]);
        const bf16x8 w1 = __builtin_bit_cast(bf16x8, fb[S][1]);
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w0, __builtin_bit_cast(bf16x8, a0[t]), acc[t], 0, 0, 0);
        // second half of k: fetched only now, into the registers the first half has left
        __builtin_amdgcn_sched_barrier(0);
        uint4 a1[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) a1[t] = *reinterpret_cast<const uint4*>(pa1 + t * 4096);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1, __builtin_bit_cast(bf16x8, a1[t]), acc[t], 0, 0, 0);
        asm volatile("" ::: "memory");
        publish_done(u_n);
        if (last) {
            epilogue(j);
            zero_acc();
            ++j;
        }
        idx = idx_n;
        item = item_n;
        u_base = u_base_n;
        u = u_n;
    };
    auto run = [&](auto SMALL_) __attribute__((always_inline)) {
        while (true) {
            do_item(std::integral_constant<int, 0>{}, SMALL_);
            if (j == ntiles) break;
            do_item(std::integral_constant<int, 1>{}, SMALL_);
            if (j == ntiles) break;
            do_item(std::integral_constant<int, 2>{}, SMALL_);
            if (j == ntiles) break;
        }
    };
    static_assert(L == 2, "the item loop is unrolled by L + 1 = 3");
    if (small) run(std::true_type{});
    else run(std::false_type{});
    publish_done(0x7fffffff);
    copy_rest();
}

}  // namespace pbs
