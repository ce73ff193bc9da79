// C ABI of libpbs_hip.so: argument checks, tile-shape choice and kernel launches.
#include "../../include/pbs_hip.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <mutex>

#include "pbs_common.h"
#include "pbs_dds.h"
#include "pbs_dds16.h"
#include "pbs_ddsc.h"
#include "pbs_index.h"
#include "pbs_sdd.h"
#include "pbs_sdd_bf16.h"
#include "pbs_sdd_seg.h"

namespace pbs {

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Zero fill as a kernel (callers may capture the stream into a graph).
__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* p, size_t nwords) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < nwords) p[i] = 0u;
}

// Kernels that use more than 64 KB of LDS need the limit raised once per device.
template <typename K>
static int raise_lds_limit(K kernel, int bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return 0;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return (int)e;
    done.fetch_or(bit, std::memory_order_release);
    return 0;
}

template <typename T, int TRANS, int TM, int SK, int RS, int RB, int NP, int NBW = DDS_NBW, int NSL = 4>
static int launch_dds(DdsArgs g, hipStream_t stream) {
    using C = DdsCfg<T, TRANS, TM, SK, RS, RB, NP, NBW, NSL>;
    static std::atomic<uint64_t> done{0};
    auto kernel = dds_kernel<T, TRANS, TM, SK, RS, RB, NP, NBW, NSL>;
    constexpr int LDS_MAX = 160 * 1024;
    // rings (or the epilogue staging) plus this group's plan records
    const size_t lds = (size_t)C::WORK_BYTES + (size_t)g.group_ints * sizeof(int);
    if (lds > (size_t)LDS_MAX) return PBS_ERR_TOO_LARGE;
    if (int rc = raise_lds_limit(kernel, LDS_MAX, done)) return rc;
    g.m_tiles = (g.M + C::BM - 1) / C::BM;
    const long long tiles = (long long)g.m_tiles * g.n_groups * C::NSUB;
    if (tiles > (1ll << 30)) return PBS_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kernel, dim3(xcd_grid((int)tiles)), dim3(C::NT), lds, stream, g);
    return (int)hipGetLastError();
}

// ---- wide-tile persistent bf16 kernel ----
// The plan buffer holds the narrow plan first, then (when k is a multiple of 64) the wide one.
// The narrow plan exists in four versions that differ in how many block columns of the result a
// group of 8 places holds (8, 7, 6 or 5; the other places stay empty): one workgroup runs per CU, so a
// launch whose tiles number 192 leaves a quarter of the chip idle, while the same columns in groups
// of 6 make 256 tiles of three quarters the work each.  Which version a launch uses depends on the
// token count, which is not known when the plan is built.
constexpr int DDS_NWIDTHS = 4;
constexpr int DDS_WIDTHS[DDS_NWIDTHS] = {8, 7, 6, 5};
static_assert(DDS_WIDTHS[DDS_NWIDTHS - 1] == DDS_MIN_WIDTH, "dds_slots_kernel sizes its table for the narrowest group");
static inline size_t narrow_groups(int n, int wi) { return ((size_t)(n / 32) + DDS_WIDTHS[wi] - 1) / DDS_WIDTHS[wi]; }
static inline size_t narrow_plan_bytes_w(int n, int k, int wi) {
    return narrow_groups(n, wi) * dds_plan_group_ints(k / 32) * sizeof(int);
}
static inline size_t slot_table_bytes_w(int n, int wi) {   // the block column in every place of every group
    return ((narrow_groups(n, wi) * DDS_NB * sizeof(int)) + 63) / 64 * 64;
}
// Plan buffer: [narrow plan, 8 columns per group][wide plan][slot table, 8][narrow 7][slots 7][narrow 6][slots 6]
// [narrow 5][slots 5].
static inline size_t narrow_plan_bytes(int n, int k) { return narrow_plan_bytes_w(n, k, 0); }
static inline size_t slot_table_bytes(int n) { return slot_table_bytes_w(n, 0); }
static inline size_t wide_plan_bytes(int n, int k) {
    if (k % 64) return 0;
    const size_t groups = ((size_t)(n / 32) + D16_NB - 1) / D16_NB;
    return (groups * dds16_plan_group_ints(k / 32) + D16_SEQ_INTS) * sizeof(int);
}

static inline size_t narrow_plan_offset(int n, int k, int wi) {
    if (wi == 0) return 0;
    size_t off = narrow_plan_bytes(n, k) + wide_plan_bytes(n, k) + slot_table_bytes(n);
    for (int i = 1; i < wi; ++i) off += narrow_plan_bytes_w(n, k, i) + slot_table_bytes_w(n, i);
    return off;
}
static inline size_t slot_table_offset(int n, int k, int wi) {
    if (wi == 0) return narrow_plan_bytes(n, k) + wide_plan_bytes(n, k);
    return narrow_plan_offset(n, k, wi) + narrow_plan_bytes_w(n, k, wi);
}
// ... and behind all of those the plan of the kernel with one block column per wave (pbs_ddsc.h), where it can
// apply: [column table][per-group lists][the table 0, 1, 2, ...].
static inline size_t column_plan_offset(int n, int k) {
    return narrow_plan_offset(n, k, DDS_NWIDTHS - 1) + narrow_plan_bytes_w(n, k, DDS_NWIDTHS - 1) +
           slot_table_bytes_w(n, DDS_NWIDTHS - 1);
}
static inline int column_groups(int n) { return (n / 32 + DC_NB - 1) / DC_NB; }
static inline size_t column_table_bytes(int n) { return ((size_t)column_groups(n) * DC_NB * sizeof(int) + 63) / 64 * 64; }
static inline size_t column_plan_bytes(int n, int k) {
    // k-pairs, and the lists of a group of 16 columns must fit the kernel's LDS area (16 * k / 32 items)
    if ((k % 64) || DC_NB * (k / 32) > DC_ITEMS_LDS) return 0;
    return column_table_bytes(n) + ((size_t)column_groups(n) * ddsc_plan_group_ints(k / 32) + DC_SEQ_INTS) * sizeof(int);
}
static inline size_t all_plan_bytes(int n, int k) { return column_plan_offset(n, k) + column_plan_bytes(n, k); }

constexpr int D16_TM = 2, D16_RS = 3, D16_RB = 32, D16_NP = 4;
constexpr double DDSC_MIN_BLOCKS_PER_COLUMN = 32.0;
constexpr int DDSC_WIDE_RESULT = 2048;

// Whether the wide kernel serves this problem: k-pairs need k % 64 == 0, the plan records of a group
// must fit in LDS beside the rings, and there must be enough tiles to give every CU one.
static bool wide_kernel_fits(long long M, int n, int k) {
    using C = D16Cfg<D16_TM, D16_RS, D16_RB, D16_NP>;
    if (k % 64) return false;
    const size_t lds = (size_t)C::WORK_BYTES + dds16_plan_group_ints(k / 32) * sizeof(int);
    if (lds > 160 * 1024) return false;
    const long long tiles = ((M + C::BM - 1) / C::BM) * ((n / 32 + D16_NB - 1) / D16_NB);
    return tiles >= 256;
}

template <int TRANS>
static int launch_dds16(const DdsArgs& g, hipStream_t stream) {
    using C = D16Cfg<D16_TM, D16_RS, D16_RB, D16_NP>;
    static std::atomic<uint64_t> done{0};
    auto kernel = dds16_kernel<TRANS, D16_TM, D16_RS, D16_RB, D16_NP>;
    D16Args a;
    a.a = g.a;
    a.data = g.data;
    a.plan = reinterpret_cast<const int*>(reinterpret_cast<const unsigned char*>(g.plan) + narrow_plan_bytes(g.N, g.K));
    a.bias = g.bias;
    a.out = g.out;
    a.M = g.M;
    a.N = g.N;
    a.K = g.K;
    a.nnz = g.nnz;
    a.m_tiles = (g.M + C::BM - 1) / C::BM;
    a.n_groups = (g.N / 32 + D16_NB - 1) / D16_NB;
    a.group_ints = (int)dds16_plan_group_ints(g.K / 32);
    a.seq = a.plan + (size_t)a.n_groups * a.group_ints;
    // about one workgroup per CU, each walking the token tiles p, p + P, ... of its column group
    int P = 256 / a.n_groups;
    if (P < 1) P = 1;
    if (P > a.m_tiles) P = a.m_tiles;
    a.wg_per_group = P;
    const size_t lds = (size_t)C::WORK_BYTES + (size_t)a.group_ints * sizeof(int);
    if (int rc = raise_lds_limit(kernel, 160 * 1024, done)) return rc;
    const long long grid = 8ll * a.n_groups * ((P + 7) / 8);
    if (grid > (1ll << 30)) return PBS_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(C::NT), lds, stream, a);
    return (int)hipGetLastError();
}

// ---- bf16 kernel with one block column per wave ----
constexpr int DDSC_RS = 8;

// PBS_COLUMN_KERNEL = 0: never use it; 1: whenever it can run; unset: where it is the faster one.
static int column_kernel_wish() {
    const char* e = std::getenv("PBS_COLUMN_KERNEL");
    if (!e || !*e) return -1;
    return e[0] == '0' ? 0 : 1;
}

struct ColumnLaunch {
    int m_tiles, n_groups, wg_per_group;
};
static inline ColumnLaunch column_launch(long long M, int n) {
    ColumnLaunch c;
    c.m_tiles = (int)((M + DC_BM - 1) / DC_BM);
    c.n_groups = column_groups(n);
    int P = 256 / c.n_groups;   // about one workgroup per CU, each walking the token tiles p, p + P, ... of its column group
    if (P < 1) P = 1;
    if (P > c.m_tiles) P = c.m_tiles;
    c.wg_per_group = P;
    return c;
}

// Whether that kernel can run this problem at all, and whether it should.  It reads a block's fragments straight
// from global memory, once per token tile, and its cost per block product is a third of the wide kernel's: 20 %
// faster at 32 blocks per column (the 4096 x 4096 layer at density 0.25), 35 % at 64.  Measured over densities
// 0.008 to 1 and results 512 to 4096 wide (16384 tokens): with a result of 2048 columns or more it is also the
// faster one for sparse patterns (4096 x 4096: 6 to 30 % at 1 to 24 blocks per column; 2048 x 2048: level at 2 to 4
// blocks per column, 5 to 13 % from 8), while results of 512 to 1024 columns stay 10 to 30 % faster in the other
// kernels until their columns hold 32 blocks.
static bool column_kernel_fits(long long M, int n, int k, int nnz, const void* bias) {
    if (!column_plan_bytes(n, k) || nnz < 1 || nnz > DC_MAX_BLOCKS || M < 1) return false;
    if (reinterpret_cast<uintptr_t>(bias) & 3u) return false;
    const ColumnLaunch c = column_launch(M, n);
    const long long tiles_per_wg = (c.m_tiles + c.wg_per_group - 1) / c.wg_per_group;
    if (tiles_per_wg * (k / 64) >= DC_SEQ_INTS) return false;   // a workgroup's steps are numbered through the table
    const int wish = column_kernel_wish();
    if (wish >= 0) return wish == 1;
    if ((long long)c.m_tiles * c.n_groups < 256) return false;
    const double per_column = (double)nnz / (n / 32);
    if (per_column >= DDSC_MIN_BLOCKS_PER_COLUMN) return true;
    // wide results (at least four groups of 16 block columns): from 16 blocks per column, and from 2 when the contraction
    // is long enough for the ring to fill (16 k-pairs)
    if (n >= DDSC_WIDE_RESULT && per_column >= 16.0) return true;
    return n >= DDSC_WIDE_RESULT && k >= 1024 && per_column >= 2.0;
}

// FM: the blocks are given in fragment order (the forward product's copy) instead of [n][k] as stored
template <bool FM>
static int launch_ddsc(const DdsArgs& g, const void* data_nk, hipStream_t stream) {
    using C = DdscCfg<DDSC_RS>;
    static std::atomic<uint64_t> done{0};
    auto kernel = ddsc_kernel<DDSC_RS, FM>;
    const ColumnLaunch c = column_launch(g.M, g.N);
    DdscArgs a;
    a.a = g.a;
    a.data = data_nk;
    a.plan = reinterpret_cast<const int*>(reinterpret_cast<const unsigned char*>(g.plan) + column_plan_offset(g.N, g.K) +
                                          column_table_bytes(g.N));
    a.bias = g.bias;
    a.out = g.out;
    a.M = g.M;
    a.N = g.N;
    a.K = g.K;
    a.nnz = g.nnz;
    a.m_tiles = c.m_tiles;
    a.n_groups = c.n_groups;
    a.group_ints = (int)ddsc_plan_group_ints(g.K / 32);
    a.seq = a.plan + (size_t)a.n_groups * a.group_ints;
    a.wg_per_group = c.wg_per_group;
    if (int rc = raise_lds_limit(kernel, 160 * 1024, done)) return rc;
    const long long grid = 8ll * a.n_groups * ((c.wg_per_group + 7) / 8);
    if (grid > (1ll << 30)) return PBS_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(C::NT), C::LDS_BYTES, stream, a);
    return (int)hipGetLastError();
}

// Tile shapes: 256 tokens x 8 block columns, 128 x 8, or 128 x 4 (twice as many, half as wide tiles).
// One workgroup runs per CU, so a launch takes ceil(tiles / 256) rounds of one tile time each; the shape
// with the smallest rounds x tile area wins (smaller tiles move more operand bytes per product, hence the
// small handicaps), e.g. 384 tiles of 128 x 8 take two rounds, of which the second is half empty, while
// the same problem in 768 tiles of 128 x 4 takes three full rounds of half the length.  A shape whose
// rings and plan records do not fit in LDS (very long contractions) is skipped.
// bf16 steps cover two k-blocks (the matrix cores go through a k-block 16x faster than in fp32).
template <typename T, int TRANS>
static int dispatch_dds(const DdsArgs& g, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    if constexpr (sizeof(T) == 2) {
        if (column_kernel_fits(g.M, g.N, g.K, g.nnz, g.bias)) {
            // the kernel wants every block with k along its rows: as stored for TRANS, a transposed copy otherwise
            if constexpr (TRANS) return launch_ddsc<false>(g, g.data, stream);
            const size_t need = (size_t)g.nnz * 2048;
            if (workspace && workspace_bytes >= need && aligned16(workspace)) {
                hipLaunchKernelGGL(transpose_blocks_kernel, dim3((unsigned)((g.nnz + 3) / 4)), dim3(256), 0, stream,
                                   static_cast<const uint16_t*>(g.data), static_cast<uint16_t*>(workspace), g.nnz);
                if (int rc = (int)hipGetLastError()) return rc;
                return launch_ddsc<true>(g, workspace, stream);
            }
        }
        if (wide_kernel_fits(g.M, g.N, g.K)) return launch_dds16<TRANS>(g, stream);
    }
    // shapes: 0 = 256 x 8 (4 token slices x 2 column halves), 1 = 128 x 8, 2 = 128 x 4,
    //         3 = 256 x 8 with 8 token slices (every wave has all 8 columns; fp32 only: 8 accumulators of fp32
    //             fragments fit the registers, and balanced waves are worth more than the larger fragments cost)
    //         fp32 shapes 1 to 3 have four copy waves beside the eight compute waves (their registers allow three
    //         waves per SIMD): a compute wave that also issues the DMA spends 900 to 1400 cycles of every step on
    //         it, at the start of the step when no wave of its SIMD has products in flight (4096 x 4096 forward
    //         1.37 -> 1.27 ms).  Shape 0 needs 200 registers per lane and keeps copying with its compute waves.
    //         4 = 128 x 4 with one k-block per step (fp32 only).  The fp32 shapes of 128 tokens take two k-blocks
    //             per step in two ring stages: their steps are short (a k-block is one or two block products per
    //             wave), so a barrier per k-block costs them a fifth of their time (768 -> 3072 input gradient at
    //             4096 tokens 0.142 -> 0.116 ms); shape 4 needs half the LDS and is what very long contractions
    //             fall through to.
    // widths: 8, 7, 6 or 5 of a tile's 8 (4) places hold a block column.  A tile's time falls with the columns it
    //         holds, though not in proportion (its panel traffic and per-step overhead stay); bf16 tiles are
    //         bound by their operand stream rather than by the matrix cores and gain less.
    constexpr int NSHAPES = sizeof(T) == 4 ? 5 : 3;
    constexpr int NCAND = NSHAPES * DDS_NWIDTHS;
    const double area[5] = {2048.0, 1024.0 * 1.04, 512.0 * 1.10, 2048.0 * 0.8, 512.0 * 1.35};
    const double fixed = sizeof(T) == 4 ? 0.15 : 0.35;   // share of a tile's time that does not depend on its columns
    double cost[NCAND];
    int order[NCAND];
    for (int wi = 0; wi < DDS_NWIDTHS; ++wi) {
        const long long groups = (long long)narrow_groups(g.N, wi);
        // of the widths that give the same number of groups only the narrowest (most even) is tried
        const bool useful = wi == 0 || (groups > (long long)narrow_groups(g.N, 0) &&
                                        (wi == DDS_NWIDTHS - 1 || groups != (long long)narrow_groups(g.N, wi + 1)));
        const long long tiles[5] = {
            (long long)((g.M + 255) / 256) * groups,
            (long long)((g.M + 127) / 128) * groups,
            (long long)((g.M + 127) / 128) * groups * 2,
            (long long)((g.M + 255) / 256) * groups,
            (long long)((g.M + 127) / 128) * groups * 2,
        };
        for (int c = 0; c < NSHAPES; ++c) {
            const int i = wi * NSHAPES + c;
            order[i] = i;
            cost[i] = useful ? (double)((tiles[c] + 255) / 256) * area[c] * (fixed + (1.0 - fixed) * DDS_WIDTHS[wi] / 8.0) * (1.0 + 0.01 * wi)
                             : 1e300;
        }
    }
    for (int i = 0; i < NCAND; ++i)
        for (int j = i + 1; j < NCAND; ++j)
            if (cost[order[j]] < cost[order[i]]) {
                const int t = order[i];
                order[i] = order[j];
                order[j] = t;
            }
    int rc = PBS_ERR_TOO_LARGE;
    for (int i = 0; i < NCAND && rc == PBS_ERR_TOO_LARGE; ++i) {
        if (cost[order[i]] >= 1e300) break;
        const int wi = order[i] / NSHAPES, c = order[i] % NSHAPES;
        DdsArgs gw = g;
        gw.plan = reinterpret_cast<const int*>(reinterpret_cast<const unsigned char*>(g.plan) + narrow_plan_offset(g.N, g.K, wi));
        gw.n_groups = (int)narrow_groups(g.N, wi);
        if constexpr (sizeof(T) == 4) {
            rc = c == 0 ? launch_dds<T, TRANS, 2, 1, 3, 8, 0>(gw, stream)
                 : c == 1 ? launch_dds<T, TRANS, 1, 2, 2, 16, 4>(gw, stream)
                 : c == 2 ? launch_dds<T, TRANS, 1, 2, 2, 16, 4, 2>(gw, stream)
                 : c == 3 ? launch_dds<T, TRANS, 1, 1, 3, 8, 4, 8, 8>(gw, stream)
                          : launch_dds<T, TRANS, 1, 1, 3, 8, 0, 2>(gw, stream);
        } else {
            rc = c == 0 ? launch_dds<T, TRANS, 2, 2, 3, 16, 4>(gw, stream)
                 : c == 1 ? launch_dds<T, TRANS, 1, 2, 3, 16, 4>(gw, stream)
                          : launch_dds<T, TRANS, 1, 2, 3, 16, 4, 2>(gw, stream);
        }
    }
    return rc;
}

// ---- sparse-output product ----
// fp32: equal shares of the blocks of a band of 16 block rows, 16-token chunks by DMA (pbs_sdd_seg.h); rectangles
// of 8 x 8 block positions staged through registers (pbs_sdd.h) where that kernel does not apply.
// bf16: 16 x 16 rectangles, 32-token chunks by DMA.
struct SddShapeF32 {
    int SR, SC, QW;
};
constexpr int SDD_F32_NSHAPES = 1;
constexpr SddShapeF32 SDD_F32_SHAPES[SDD_F32_NSHAPES] = {{8, 8, 8}};
constexpr int SDD_F32_NW = 8, SDD_F32_TC = 16;
struct SddShapeBf16 {
    static constexpr int SR = 16, SC = 16, QW = 10, TC = 32, NS = 2, NW = 8;
};

struct SddPlan {
    int tiles_r, tiles_c, nsplit, tokens_per_split;
    int shape;   // fp32: index into SDD_F32_SHAPES, or SDD_F32_SEGMENTS
    int segs;    // segment kernel: shares per row band
};
constexpr int SDD_F32_SEGMENTS = SDD_F32_NSHAPES;
constexpr int SEG_SR = 16, SEG_QW = 9;
constexpr int SEG_NSC = 2;
constexpr int SEG_SC[SEG_NSC] = {16, 20};   // X panel widths of the two builds of the segment kernel

static SddPlan plan_sdd(long long M, int N, int K, int SR, int SC, int TC) {
    SddPlan p;
    p.shape = 0;
    p.segs = 0;
    p.tiles_r = (N / 32 + SR - 1) / SR;
    p.tiles_c = (K / 32 + SC - 1) / SC;
    const long long tiles = (long long)p.tiles_r * p.tiles_c;
    const long long chunks = (M + TC - 1) / TC;
    // Aim at one workgroup per CU and never slightly more (the kernels' registers and LDS allow one
    // workgroup per CU, so 257 workgroups take twice as long as 256); keep at least 8 chunks per slice.
    long long want = 256 / tiles;
    long long cap = chunks / 8;
    if (cap < 1) cap = 1;
    if (want > cap) want = cap;
    if (want < 1) want = 1;
    const long long chunks_per = (chunks + want - 1) / want;
    p.nsplit = (int)((chunks + chunks_per - 1) / chunks_per);
    if (p.nsplit < 1) p.nsplit = 1;
    p.tokens_per_split = (int)(chunks_per * TC);
    return p;
}
// fp32: which kernel, and how the work is cut.  A workgroup's time per chunk of tokens is set by its busiest
// wave, i.e. by rounds = ceil(blocks of the workgroup / 8), and the launch ends with its slowest workgroup.  The
// estimate for either kernel is chunks per workgroup x (rounds + a half for the chunk's staging and barriers).
// Rectangles: the fullest of the rectangles expected under a uniform pattern of the given density (33 blocks
// on 8 waves cost 5 rounds for 4.1 rounds of work).
static SddPlan plan_sdd_f32(long long M, int N, int K, long long nnz) {
    const SddShapeF32 sh = SDD_F32_SHAPES[0];
    SddPlan best = plan_sdd(M, N, K, sh.SR, sh.SC, SDD_F32_TC);
    const double positions = (double)(N / 32) * (double)(K / 32);
    const double d = positions > 0 ? (double)nnz / positions : 0.0;
    double best_cost;
    {
        const int sr = N / 32 < sh.SR ? N / 32 : sh.SR, sc = K / 32 < sh.SC ? K / 32 : sh.SC;
        const double mean = sr * sc * d;
        const double full = (double)((N / 32) / sh.SR > 0 ? (N / 32) / sh.SR : 1) * ((K / 32) / sh.SC > 0 ? (K / 32) / sh.SC : 1);
        const double spread = std::sqrt(mean * (1.0 - d)) * std::sqrt(2.0 * std::log(full < 2.0 ? 2.0 : full));
        double fullest = mean + spread;
        if (fullest > sr * sc) fullest = sr * sc;
        double rounds = std::ceil(fullest / SDD_F32_NW);
        if (rounds < 1.0) rounds = 1.0;
        if (fullest > sh.QW * SDD_F32_NW) rounds *= 2.0;   // a second pass over the tokens
        best_cost = (double)best.tokens_per_split / SDD_F32_TC * (rounds + 0.5);
    }
    // Equal shares of each row band's blocks (pbs_sdd_seg.h): every workgroup does `rounds` products per chunk.
    // A share of 8 x rounds blocks spans about that many / (rows x density) block columns, which must fit the
    // kernel's X panel; bands differ a little in their block counts, so the shares are sized for a band two
    // standard deviations above the mean.  Of the feasible rounds the one with the smallest chunks x rounds wins.
    const int nblk_r = N / 32, ncols = K / 32;
    for (int v = 0; v < SEG_NSC; ++v) {
        // the histogram of a band's block columns borrows the stage buffers
        const int max_cols = 2 * 16 * (SEG_SR + SEG_SC[v]) * 128 / 4 - 64;
        if (ncols > max_cols || nnz <= 0 || d <= 0.0) continue;
        const int bands = (nblk_r + SEG_SR - 1) / SEG_SR;
        const int rows_per_band = (nblk_r + bands - 1) / bands;
        const double n_band = (double)nnz * rows_per_band / nblk_r;
        const double heavy = n_band + (bands > 1 ? 2.0 * std::sqrt(n_band * (1.0 - d)) : 0.0);
        const long long chunks = (M + SDD_F32_TC - 1) / SDD_F32_TC;
        for (int q = 1; q <= SEG_QW; ++q) {
            const double share = 8.0 * q;
            if (share / (rows_per_band * d) + 2.0 > SEG_SC[v]) break;   // wider than the X panel
            long long segs = (long long)std::ceil(heavy / share);
            if (segs < 1) segs = 1;
            const long long wgs1 = (long long)bands * segs;
            long long want = 256 / wgs1, cap = chunks / 8;
            if (cap < 1) cap = 1;
            if (want > cap) want = cap;
            if (want < 1) want = 1;
            const long long chunks_per = (chunks + want - 1) / want;
            const long long nsplit = (chunks + chunks_per - 1) / chunks_per;
            const double waves_of_wgs = std::ceil((double)(wgs1 * nsplit) / 256.0);
            const double rounds = std::ceil(n_band / segs / 8.0);
            // the wider panel costs a few per cent (more bytes staged per chunk)
            const double cost = (double)chunks_per * (rounds + 0.5) * waves_of_wgs * (1.0 + 0.04 * v);
            if (cost < best_cost) {
                best_cost = cost;
                best.shape = SDD_F32_SEGMENTS + v;
                best.tiles_r = bands;
                best.tiles_c = 1;
                best.segs = (int)segs;
                best.nsplit = (int)nsplit;
                best.tokens_per_split = (int)(chunks_per * SDD_F32_TC);
            }
        }
    }
    return best;
}
static SddPlan plan_sdd_for(int dtype, long long M, int N, int K, long long nnz) {
    if (dtype == PBS_DTYPE_F32) return plan_sdd_f32(M, N, K, nnz);
    return plan_sdd(M, N, K, SddShapeBf16::SR, SddShapeBf16::SC, SddShapeBf16::TC);
}

template <int SHAPE>
static int launch_sdd_f32(const SddArgs& a, long long wgs, hipStream_t stream) {
    constexpr SddShapeF32 S = SDD_F32_SHAPES[SHAPE];
    using C = SddCfg<float, S.SR, S.SC, S.QW, SDD_F32_NW>;
    static_assert(C::TC == SDD_F32_TC, "plan and kernel must agree on the chunk size");
    static std::atomic<uint64_t> done{0};
    auto kernel = sdd_kernel<float, S.SR, S.SC, S.QW, SDD_F32_NW>;
    if (int rc = raise_lds_limit(kernel, C::LDS_BYTES, done)) return rc;
    hipLaunchKernelGGL(kernel, dim3(xcd_grid((int)wgs)), dim3(C::NT), C::LDS_BYTES, stream, a);
    return (int)hipGetLastError();
}

template <int V>
static int launch_sdd_seg(const SddArgs& a, long long wgs, hipStream_t stream) {
    using C = SddSegCfg<SEG_SR, SEG_SC[V], SEG_QW, SDD_F32_NW>;
    static_assert(C::MAX_COLS == 2 * 16 * (SEG_SR + SEG_SC[V]) * 128 / 4 - 64, "the plan's column limit is the kernel's");
    static_assert(C::TC == SDD_F32_TC, "plan and kernel must agree on the chunk size");
    static std::atomic<uint64_t> done{0};
    auto kernel = sdd_seg_kernel<SEG_SR, SEG_SC[V], SEG_QW, SDD_F32_NW>;
    if (int rc = raise_lds_limit(kernel, C::LDS_BYTES, done)) return rc;
    hipLaunchKernelGGL(kernel, dim3(xcd_grid((int)wgs)), dim3(C::NT), C::LDS_BYTES, stream, a);
    return (int)hipGetLastError();
}

template <typename T>
static int launch_sdd(SddArgs a, int dtype, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    const SddPlan p = plan_sdd_for(dtype, a.M, a.N, a.K, a.nnz);
    a.tiles_r = p.tiles_r;
    a.tiles_c = p.tiles_c;
    a.nsplit = p.nsplit;
    a.tokens_per_split = p.tokens_per_split;
    a.segs = p.segs;
    a.partial = nullptr;
    const size_t n = (size_t)a.nnz * 1024;
    if (p.nsplit > 1) {
        const size_t need = n * sizeof(float) * p.nsplit;
        if (!workspace || workspace_bytes < need || !aligned16(workspace)) return PBS_ERR_WORKSPACE;
        a.partial = static_cast<float*>(workspace);
    }
    const long long wgs = (long long)p.tiles_r * (p.segs > 0 ? p.segs : p.tiles_c) * p.nsplit;
    if (wgs > (1ll << 30)) return PBS_ERR_TOO_LARGE;
    if constexpr (sizeof(T) == 4) {
        const int rc = p.shape == SDD_F32_SEGMENTS ? launch_sdd_seg<0>(a, wgs, stream)
                       : p.shape == SDD_F32_SEGMENTS + 1 ? launch_sdd_seg<1>(a, wgs, stream)
                                                         : launch_sdd_f32<0>(a, wgs, stream);
        if (rc) return rc;
    } else {
        using S = SddShapeBf16;
        using C = SddBf16Cfg<S::QW, S::TC, S::NS, S::NW>;
        static_assert(C::TC == S::TC && C::SR == S::SR && C::SC == S::SC, "plan and kernel must agree");
        static std::atomic<uint64_t> done{0};
        auto kernel = sdd_bf16_kernel<S::QW, S::TC, S::NS, S::NW>;
        if (int rc = raise_lds_limit(kernel, C::LDS_BYTES, done)) return rc;
        hipLaunchKernelGGL(kernel, dim3(xcd_grid((int)wgs)), dim3(C::NT), C::LDS_BYTES, stream, a);
    }
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    if (p.nsplit > 1) {
        const unsigned grid = (unsigned)((n / 4 + 255) / 256);
        hipLaunchKernelGGL(sdd_reduce_kernel<T>, dim3(grid), dim3(256), 0, stream, a.partial, static_cast<T*>(a.out), n,
                           p.nsplit);
        rc = (int)hipGetLastError();
    }
    return rc;
}

// ---- scratch of the entry point that allocates nothing ----
// One device array per GPU, part of the library's code object: it exists on every GPU the library runs on
// from the moment the code object is loaded there until the process ends.  Host code never uses the
// array's name as an address (on the host it only stands for the symbol): the address on a device is
// asked for once, with that device current, and kept.
static __device__ __align__(256) unsigned char scratch[PBS_NOALLOC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return PBS_ERR_TOO_LARGE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return PBS_ERR_WORKSPACE;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return PBS_OK;
}

}  // namespace pbs

using namespace pbs;

extern "C" {

int pbs_abi_version(void) { return PBS_ABI_VERSION; }


const char* pbs_error_string(int code) {
    switch (code) {
        case PBS_OK: return "ok";
        case PBS_ERR_NULL_POINTER: return "pbs: null pointer argument";
        case PBS_ERR_BAD_SHAPE: return "pbs: bad shape (negative size, or a feature dimension that is not a multiple of 32)";
        case PBS_ERR_BAD_DTYPE: return "pbs: unknown dtype code";
        case PBS_ERR_MISALIGNED: return "pbs: dense/data pointers must be 16-byte aligned";
        case PBS_ERR_WORKSPACE: return "pbs: workspace missing, misaligned or too small";
        case PBS_ERR_TOO_LARGE: return "pbs: size exceeds the kernels' index range";
        case PBS_ERR_SCRATCH: return "pbs: the problem needs more scratch than the library's built-in buffer holds; use the entry point that takes a workspace";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "pbs: unknown error code";
}

int pbs_build_indices(const uint8_t* mask, const int64_t* block_ptr, int X, int Y, int nnz, int32_t* cols_a,
                      int32_t* row_start_ends_a, int32_t* rows_b, int32_t* col_start_ends_b, int32_t* blocks,
                      int32_t* status, void* stream) {
    if (X < 1 || Y < 1 || nnz < 0 || (long long)nnz > (long long)X * Y) return PBS_ERR_BAD_SHAPE;
    if ((long long)X * Y > (1ll << 30)) return PBS_ERR_TOO_LARGE;
    if (!mask || !row_start_ends_a || !col_start_ends_b || !status) return PBS_ERR_NULL_POINTER;
    if (nnz > 0 && (!cols_a || !rows_b || !blocks)) return PBS_ERR_NULL_POINTER;
    hipLaunchKernelGGL(build_indices_kernel, dim3(1), dim3(INDEX_THREADS), 0, static_cast<hipStream_t>(stream), mask,
                       block_ptr, X, Y, nnz, cols_a, row_start_ends_a, rows_b, col_start_ends_b, blocks, status);
    return (int)hipGetLastError();
}

size_t pbs_blocksparse_matmul_plan_bytes(int n, int k) {
    if (n <= 0 || k <= 0 || (n % 32) || (k % 32)) return 0;
    return all_plan_bytes(n, k);
}

int pbs_blocksparse_matmul_plan(const int32_t* ptr, const int32_t* indices, int n, int k, int nnz, void* plan,
                                size_t plan_bytes, void* stream) {
    if (n <= 0 || k <= 0 || nnz < 0 || (n % 32) || (k % 32)) return PBS_ERR_BAD_SHAPE;
    if ((long long)nnz > (long long)(n / 32) * (k / 32) || k > (1 << 24)) return PBS_ERR_TOO_LARGE;
    if (!ptr || !plan || (nnz > 0 && !indices)) return PBS_ERR_NULL_POINTER;
    if (!aligned16(plan) || plan_bytes < pbs_blocksparse_matmul_plan_bytes(n, k)) return PBS_ERR_WORKSPACE;
    for (int wi = 0; wi < DDS_NWIDTHS; ++wi) {
        const int groups = (int)narrow_groups(n, wi);
        int* slots = reinterpret_cast<int*>(static_cast<unsigned char*>(plan) + slot_table_offset(n, k, wi));
        int* narrow = reinterpret_cast<int*>(static_cast<unsigned char*>(plan) + narrow_plan_offset(n, k, wi));
        hipLaunchKernelGGL(dds_slots_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream), ptr, n / 32, groups,
                           DDS_WIDTHS[wi], slots);
        if (int rc = (int)hipGetLastError()) return rc;
        hipLaunchKernelGGL(dds_plan_kernel, dim3(groups), dim3(256), 0, static_cast<hipStream_t>(stream), ptr, indices,
                           slots, n / 32, k / 32, nnz, narrow, (int)dds_plan_group_ints(k / 32));
        if (int rc = (int)hipGetLastError()) return rc;
    }
    if (wide_plan_bytes(n, k)) {
        const int groups16 = (n / 32 + D16_NB - 1) / D16_NB;
        int* wide = reinterpret_cast<int*>(static_cast<unsigned char*>(plan) + narrow_plan_bytes(n, k));
        hipLaunchKernelGGL(dds16_plan_kernel, dim3(groups16), dim3(256), 0, static_cast<hipStream_t>(stream), ptr, indices,
                           n / 32, k / 32, nnz, wide, (int)dds16_plan_group_ints(k / 32),
                           wide + (size_t)groups16 * dds16_plan_group_ints(k / 32));
        if (int rc = (int)hipGetLastError()) return rc;
    }
    if (column_plan_bytes(n, k)) {
        const int groups = column_groups(n);
        const int group_ints = (int)ddsc_plan_group_ints(k / 32);
        int* cols = reinterpret_cast<int*>(static_cast<unsigned char*>(plan) + column_plan_offset(n, k));
        int* lists = reinterpret_cast<int*>(static_cast<unsigned char*>(plan) + column_plan_offset(n, k) + column_table_bytes(n));
        hipStream_t s = static_cast<hipStream_t>(stream);
        hipLaunchKernelGGL(ddsc_cols_kernel, dim3(1), dim3(256), 0, s, ptr, n / 32, groups, nnz, cols);
        if (int rc = (int)hipGetLastError()) return rc;
        hipLaunchKernelGGL(ddsc_plan_kernel, dim3(groups), dim3(256), 0, s, ptr, indices, cols, n / 32, k / 32, nnz, lists,
                           group_ints, lists + (size_t)groups * group_ints);
        if (int rc = (int)hipGetLastError()) return rc;
        hipLaunchKernelGGL(ddsc_plan_ahead_kernel, dim3(groups), dim3(64), 0, s, k / 32, lists, group_ints);
    }
    return (int)hipGetLastError();
}

size_t pbs_blocksparse_matmul_workspace_bytes(int64_t tokens, int n, int k, int nnz, int transpose, int dtype) {
    if (dtype != PBS_DTYPE_BF16 || !transpose || tokens <= 0 || n <= 0 || k <= 0 || nnz <= 0 || (n % 32) || (k % 32)) return 0;
    if ((long long)nnz > (long long)(n / 32) * (k / 32)) return 0;
    return column_kernel_fits(tokens, n, k, nnz, nullptr) ? (size_t)nnz * 2048 : 0;
}

int pbs_blocksparse_matmul(const void* dense_a, const void* data, const void* plan, const void* bias, void* dense_out,
                           int64_t tokens, int n, int k, int nnz, int transpose, int dtype, void* stream) {
    return pbs_blocksparse_matmul_ws(dense_a, data, plan, bias, dense_out, tokens, n, k, nnz, transpose, dtype, nullptr, 0,
                                     stream);
}

int pbs_blocksparse_matmul_ws(const void* dense_a, const void* data, const void* plan, const void* bias, void* dense_out,
                              int64_t tokens, int n, int k, int nnz, int transpose, int dtype, void* workspace,
                              size_t workspace_bytes, void* stream) {
    if (dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) return PBS_ERR_BAD_DTYPE;
    if (tokens < 0 || n <= 0 || k <= 0 || nnz < 0 || (n % 32) || (k % 32)) return PBS_ERR_BAD_SHAPE;
    if (tokens > (1ll << 30) || (long long)nnz > (long long)(n / 32) * (k / 32) || k > (1 << 24)) return PBS_ERR_TOO_LARGE;
    if (tokens == 0) return PBS_OK;
    if (!dense_a || !plan || !dense_out) return PBS_ERR_NULL_POINTER;
    if (nnz > 0 && !data) return PBS_ERR_NULL_POINTER;
    if (!aligned16(dense_a) || !aligned16(data) || !aligned16(dense_out) || !aligned16(plan)) return PBS_ERR_MISALIGNED;
    DdsArgs g;
    g.a = dense_a;
    g.data = data;
    g.plan = static_cast<const int*>(plan);
    g.bias = bias;
    g.out = dense_out;
    g.M = (int)tokens;
    g.N = n;
    g.K = k;
    g.nnz = nnz;
    g.m_tiles = 0;
    g.n_groups = (n / 32 + DDS_NB - 1) / DDS_NB;
    g.group_ints = (int)dds_plan_group_ints(k / 32);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == PBS_DTYPE_F32) {
        return transpose ? dispatch_dds<float, 0>(g, nullptr, 0, s) : dispatch_dds<float, 1>(g, nullptr, 0, s);
    }
    return transpose ? dispatch_dds<bf16_t, 0>(g, workspace, workspace_bytes, s)
                     : dispatch_dds<bf16_t, 1>(g, nullptr, 0, s);
}

size_t pbs_blocksparse_matmul_back_workspace_bytes(int64_t tokens, int out_features, int in_features, int nnz,
                                                   int dtype) {
    if (tokens <= 0 || out_features <= 0 || in_features <= 0 || nnz <= 0) return 0;
    if ((out_features % 32) || (in_features % 32)) return 0;
    if (dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) return 0;
    const SddPlan p = plan_sdd_for(dtype, tokens, out_features, in_features, nnz);
    if (p.nsplit <= 1) return 0;
    return (size_t)nnz * 1024 * sizeof(float) * p.nsplit;
}

int pbs_blocksparse_matmul_back(const void* dense_a, const void* dense_b, const int32_t* row_start_ends_a,
                                const int32_t* cols_a, void* data_out, int64_t tokens, int out_features,
                                int in_features, int nnz, int dtype, void* workspace, size_t workspace_bytes,
                                void* stream) {
    if (dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) return PBS_ERR_BAD_DTYPE;
    if (tokens < 0 || out_features <= 0 || in_features <= 0 || nnz < 0 || (out_features % 32) || (in_features % 32))
        return PBS_ERR_BAD_SHAPE;
    if (tokens > (1ll << 30) || (long long)nnz > (long long)(out_features / 32) * (in_features / 32))
        return PBS_ERR_TOO_LARGE;
    if (nnz == 0) return PBS_OK;
    if (!row_start_ends_a || !cols_a || !data_out) return PBS_ERR_NULL_POINTER;
    if (tokens > 0 && (!dense_a || !dense_b)) return PBS_ERR_NULL_POINTER;
    if (!aligned16(dense_a) || !aligned16(dense_b) || !aligned16(data_out)) return PBS_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (tokens == 0) {
        const size_t nwords = (size_t)nnz * 1024 * (dtype == PBS_DTYPE_F32 ? 4 : 2) / 4;
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((nwords + 255) / 256)), dim3(256), 0, s,
                           static_cast<uint32_t*>(data_out), nwords);
        return (int)hipGetLastError();
    }
    SddArgs a;
    a.g = dense_a;
    a.x = dense_b;
    a.ptr = row_start_ends_a;
    a.idx = cols_a;
    a.out = data_out;
    a.partial = nullptr;
    a.M = (int)tokens;
    a.N = out_features;
    a.K = in_features;
    a.nnz = nnz;
    a.tiles_r = a.tiles_c = a.nsplit = a.tokens_per_split = a.segs = 0;
    if (dtype == PBS_DTYPE_F32) return launch_sdd<float>(a, dtype, workspace, workspace_bytes, s);
    return launch_sdd<bf16_t>(a, dtype, workspace, workspace_bytes, s);
}

// ---- the reference's own signature of the sparse-output product ----
struct BackBlocksLayout {
    size_t row_ptr, cols_a, owner, a_t, b_t, inner, total;   // byte offsets into the workspace; inner = the split workspace
};
static inline size_t round256(size_t v) { return (v + 255) / 256 * 256; }
static BackBlocksLayout back_blocks_layout(int64_t tokens, int out_features, int in_features, int nnz, int dtype,
                                           int a_row_major, int b_row_major) {
    BackBlocksLayout l;
    const size_t X = out_features / 32, Y = in_features / 32, esz = dtype == PBS_DTYPE_F32 ? 4 : 2;
    size_t off = 0;
    l.row_ptr = off;
    off += round256((X + 1) * sizeof(int32_t));
    l.cols_a = off;
    off += round256((size_t)nnz * 2 * sizeof(int32_t));
    l.owner = off;
    off += round256(X * Y * sizeof(int));
    l.a_t = off;
    if (!a_row_major) off += round256((size_t)tokens * out_features * esz);
    l.b_t = off;
    if (!b_row_major) off += round256((size_t)tokens * in_features * esz);
    l.inner = off;
    off += round256(pbs_blocksparse_matmul_back_workspace_bytes(tokens, out_features, in_features, nnz, dtype));
    l.total = off;
    return l;
}

size_t pbs_blocksparse_matmul_back_blocks_workspace_bytes(int64_t tokens, int out_features, int in_features, int nnz,
                                                          int dtype, int a_row_major, int b_row_major) {
    if (tokens < 0 || out_features <= 0 || in_features <= 0 || nnz <= 0) return 0;
    if ((out_features % 32) || (in_features % 32)) return 0;
    if (dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) return 0;
    return back_blocks_layout(tokens, out_features, in_features, nnz, dtype, a_row_major, b_row_major).total;
}

int pbs_blocksparse_matmul_back_blocks(const void* dense_a, int a_row_major, const void* dense_b, int b_row_major,
                                       void* data_out, int64_t tokens, int out_features, int in_features,
                                       const int32_t* blocks, int nnz, int dtype, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    if (dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) return PBS_ERR_BAD_DTYPE;
    if (tokens < 0 || out_features <= 0 || in_features <= 0 || nnz < 0 || (out_features % 32) || (in_features % 32))
        return PBS_ERR_BAD_SHAPE;
    if (tokens > (1ll << 30) || (long long)nnz > (long long)(out_features / 32) * (in_features / 32))
        return PBS_ERR_TOO_LARGE;
    if (nnz == 0) return PBS_OK;
    if (!blocks || !data_out) return PBS_ERR_NULL_POINTER;
    if (tokens > 0 && (!dense_a || !dense_b)) return PBS_ERR_NULL_POINTER;
    if (!aligned16(dense_a) || !aligned16(dense_b) || !aligned16(data_out)) return PBS_ERR_MISALIGNED;
    const BackBlocksLayout l = back_blocks_layout(tokens, out_features, in_features, nnz, dtype, a_row_major, b_row_major);
    if (!workspace || workspace_bytes < l.total || !aligned16(workspace)) return PBS_ERR_WORKSPACE;
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int X = out_features / 32, Y = in_features / 32;
    int32_t* row_ptr = reinterpret_cast<int32_t*>(ws + l.row_ptr);
    int32_t* cols_a = reinterpret_cast<int32_t*>(ws + l.cols_a);
    int* owner = reinterpret_cast<int*>(ws + l.owner);
    const long long positions = (long long)X * Y;
    hipLaunchKernelGGL(blocks_owner_clear_kernel, dim3((unsigned)((positions + 255) / 256)), dim3(256), 0, s, owner, positions);
    hipLaunchKernelGGL(blocks_owner_kernel, dim3((unsigned)((nnz + 255) / 256)), dim3(256), 0, s, blocks, nnz, X, Y, owner);
    hipLaunchKernelGGL(csr_from_owner_kernel, dim3(1), dim3(INDEX_THREADS), 0, s, owner, X, Y, cols_a, row_ptr);
    if (int rc = (int)hipGetLastError()) return rc;
    // an operand given with the tokens along its rows' direction ([features, tokens]) is brought to [tokens, features]
    auto to_row_major = [&](const void* src, size_t off, int features) -> int {
        const dim3 grid((unsigned)((tokens + 31) / 32), (unsigned)((features + 31) / 32));
        if (dtype == PBS_DTYPE_F32)
            hipLaunchKernelGGL(transpose_dense_kernel<uint32_t>, grid, dim3(256), 0, s, static_cast<const uint32_t*>(src),
                               reinterpret_cast<uint32_t*>(ws + off), (long long)features, (long long)tokens);
        else
            hipLaunchKernelGGL(transpose_dense_kernel<uint16_t>, grid, dim3(256), 0, s, static_cast<const uint16_t*>(src),
                               reinterpret_cast<uint16_t*>(ws + off), (long long)features, (long long)tokens);
        return (int)hipGetLastError();
    };
    const void* a = dense_a;
    const void* b = dense_b;
    if (!a_row_major && tokens > 0) {
        if (int rc = to_row_major(dense_a, l.a_t, out_features)) return rc;
        a = ws + l.a_t;
    }
    if (!b_row_major && tokens > 0) {
        if (int rc = to_row_major(dense_b, l.b_t, in_features)) return rc;
        b = ws + l.b_t;
    }
    return pbs_blocksparse_matmul_back(a, b, row_ptr, cols_a, data_out, tokens, out_features, in_features, nnz, dtype,
                                       ws + l.inner, l.total - l.inner, stream);
}

size_t pbs_blocksparse_matmul_back_noalloc_max_bytes(void) { return PBS_NOALLOC_SCRATCH_BYTES; }

int pbs_blocksparse_matmul_back_noalloc_init(void) {
    void* ws = nullptr;
    return scratch_of_current_device(&ws);
}

int pbs_blocksparse_matmul_back_noalloc(const void* dense_a, const void* dense_b, const int32_t* row_start_ends_a,
                                        const int32_t* cols_a, void* data_out, int64_t tokens, int out_features,
                                        int in_features, int nnz, int dtype, void* stream) {
    // what pbs_blocksparse_matmul_back would ask the caller for (0 for arguments it is going to reject itself)
    const size_t need = pbs_blocksparse_matmul_back_workspace_bytes(tokens, out_features, in_features, nnz, dtype);
    if (need > (size_t)PBS_NOALLOC_SCRATCH_BYTES) return PBS_ERR_SCRATCH;
    void* ws = nullptr;
    if (need > 0) {
        if (int rc = scratch_of_current_device(&ws)) return rc;
    }
    return pbs_blocksparse_matmul_back(dense_a, dense_b, row_start_ends_a, cols_a, data_out, tokens, out_features,
                                       in_features, nnz, dtype, ws, need, stream);
}

int pbs_protocol_failures(unsigned* count) {
    if (!count) return PBS_ERR_NULL_POINTER;
    return (int)hipMemcpyFromSymbol(count, HIP_SYMBOL(g_protocol_failures), sizeof(unsigned), 0, hipMemcpyDeviceToHost);
}

const char* pbs_blocksparse_matmul_kernel_name(int64_t tokens, int n, int k, int nnz, int transpose, int dtype,
                                               int with_workspace) {
    if ((dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) || tokens <= 0 || n <= 0 || k <= 0 || (n % 32) || (k % 32)) return "";
    if (dtype == PBS_DTYPE_BF16) {
        if ((!transpose || with_workspace) && column_kernel_fits(tokens, n, k, nnz, nullptr)) return "ddsc_kernel";
        if (wide_kernel_fits(tokens, n, k)) return "dds16_kernel";
    }
    return "dds_kernel";
}

const char* pbs_blocksparse_matmul_back_kernel_name(int64_t tokens, int out_features, int in_features, int nnz, int dtype) {
    if ((dtype != PBS_DTYPE_F32 && dtype != PBS_DTYPE_BF16) || tokens <= 0 || out_features <= 0 || in_features <= 0 ||
        nnz <= 0 || (out_features % 32) || (in_features % 32))
        return "";
    const SddPlan p = plan_sdd_for(dtype, tokens, out_features, in_features, nnz);
    if (dtype == PBS_DTYPE_BF16) return p.nsplit > 1 ? "sdd_bf16_kernel + sdd_reduce_kernel" : "sdd_bf16_kernel";
    if (p.shape >= SDD_F32_SEGMENTS) return p.nsplit > 1 ? "sdd_seg_kernel + sdd_reduce_kernel" : "sdd_seg_kernel";
    return p.nsplit > 1 ? "sdd_kernel + sdd_reduce_kernel" : "sdd_kernel";
}

}  // extern "C"
