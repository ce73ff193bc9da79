// dense x block-sparse -> dense (forward Y = X.W^T and input gradient dX = dY.W).
//
// One workgroup owns a BM-token x NB-block-column tile of the result (block columns of the
// *result*: block rows of W for the forward, block columns of W for dX).  It merges the NB sorted
// block lists of its tile into one list of steps -- the k-blocks any of them touches -- in LDS,
// then walks the steps: the BM x 32 dense operand panel of the step and the (at most NB) packed
// blocks are staged in LDS, double buffered through registers, and each wave issues MFMAs only
// for the (block column, step) pairs that exist.
#pragma once
#include "pbs_common.h"

namespace pbs {

struct DdsArgs {
    const void* a;         // [M, K] row-major
    const void* data;      // [nnz*32, 32]
    const int32_t* ptr;    // [N/32 + 1]
    const int32_t* idx;    // [nnz][2] = (k-block, data block)
    const void* bias;      // nullptr or [N]
    void* out;             // [M, N] row-major
    int M, N, K, nnz;
    int m_tiles, n_groups;
};

// TRANS = 0: B[k][n] = block[k*32 + n]   (forward: the packed block is W_block^T = [in][out])
// TRANS = 1: B[k][n] = block[n*32 + k]   (dX: contraction runs along the packed block's rows)
template <typename T, int TRANS, int TM, int TN, int WGM, int WGN>
struct DdsCfg {
    using E = Elem<T>;
    static constexpr int NW = WGM * WGN;
    static constexpr int NT = NW * 64;
    static constexpr int BM = WGM * TM * 32;
    static constexpr int NB = WGN * TN;
    static constexpr int SEG = 256;                      // k-blocks merged per table build
    static constexpr int ROWB = 32 * E::ESZ;             // bytes of one 32-wide operand row
    static constexpr int PITCH = ROWB + 16;              // padded: 16-byte reads of 16 rows hit 16 bank groups
    static constexpr int CPR = ROWB / 16;                // 16-byte chunks per row
    static constexpr int A_BYTES = BM * PITCH;
    static constexpr int NA = BM * CPR / NT;             // A chunks per thread per step
    // B block in LDS: TRANS=1 keeps [n][k] rows (k contiguous) with the padded pitch; TRANS=0 keeps
    // [k][n] for fp32 (read one word per k) and k-pair-interleaved words [k/2][n] for bf16.
    static constexpr int BLK_BYTES = TRANS ? 32 * PITCH : 1024 * E::ESZ;
    static constexpr int B_BYTES = NB * BLK_BYTES;
    static constexpr int CPB = 1024 * E::ESZ / 16;       // 16-byte chunks per packed block
    static constexpr int NBC = NB * CPB / NT;            // B chunks per thread per step
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int TBL_BYTES = (SEG * NB + SEG + NB + 1 + 3) * 4;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES + TBL_BYTES;
    static_assert((BM * CPR) % NT == 0, "A staging must divide evenly");
    static_assert((NB * CPB) % NT == 0, "B staging must divide evenly");
    static_assert(E::ESZ == 4 || TRANS == 1 || NBC % 2 == 0, "bf16 forward stages row pairs");
    static_assert(STAGE_BYTES % 16 == 0, "stage alignment");
};

template <typename T, int TRANS, int TM, int TN, int WGM, int WGN>
__global__ __launch_bounds__(WGM* WGN * 64) void dds_kernel(DdsArgs g) {
    using C = DdsCfg<T, TRANS, TM, TN, WGM, WGN>;
    using E = typename C::E;
    constexpr int NT = C::NT, NB = C::NB, SEG = C::SEG, NQ = E::NQ;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* stage0 = smem;
    int* s_tbl = reinterpret_cast<int*>(smem + 2 * C::STAGE_BYTES);  // [SEG][NB] data block or -1
    int* s_steps = s_tbl + SEG * NB;                                 // [SEG] local k-block of each step
    int* s_ptr = s_steps + SEG;                                      // [NB+1]
    int* s_nsteps = s_ptr + NB + 1;

    const int tile = xcd_tile_id(blockIdx.x, g.m_tiles * g.n_groups);
    if (tile < 0) return;
    const int mt = tile / g.n_groups;
    const int ng = tile % g.n_groups;
    const int m0 = mt * C::BM;
    const int nb0 = ng * NB;
    const int nblk_n = g.N / 32;
    const int KB = g.K / 32;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WGN;
    const int wn = wave % WGN;
    const int lrow = lane & 31;
    const int h = lane >> 5;

    const unsigned char* A = static_cast<const unsigned char*>(g.a);
    const unsigned char* D = static_cast<const unsigned char*>(g.data);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    if (tid <= NB) {
        int nb = nb0 + tid;
        s_ptr[tid] = g.ptr[nb < nblk_n ? nb : nblk_n];
    }
    __syncthreads();
    const int e_begin = s_ptr[0];
    const int e_end = s_ptr[NB];

    uint4 ra[C::NA];
    uint4 rb[C::NBC];

    for (int seg0 = 0; seg0 < KB; seg0 += SEG) {
        // ---- merge the NB block lists restricted to k-blocks [seg0, seg0+SEG) ----
        for (int i = tid; i < SEG * NB; i += NT) s_tbl[i] = -1;
        __syncthreads();
        for (int e = e_begin + tid; e < e_end; e += NT) {
            const int kb = g.idx[2 * e] - seg0;
            const int b = g.idx[2 * e + 1];
            if (kb >= 0 && kb < SEG && kb + seg0 < KB && b >= 0 && b < g.nnz) {
                int nl = 0;
#pragma unroll
                for (int i = 1; i < NB; ++i) nl += (e >= s_ptr[i]) ? 1 : 0;
                s_tbl[kb * NB + nl] = b;
            }
        }
        __syncthreads();
        if (wave == 0) {
            int running = 0;
            for (int base = 0; base < SEG; base += 64) {
                const int kbl = base + lane;
                bool any = false;
#pragma unroll
                for (int i = 0; i < NB; ++i) any |= (s_tbl[kbl * NB + i] >= 0);
                const unsigned long long m = __ballot(any);
                if (any) s_steps[running + __popcll(m & ((1ull << lane) - 1ull))] = kbl;
                running += __popcll(m);
            }
            if (lane == 0) *s_nsteps = running;
        }
        __syncthreads();
        const int ns = *s_nsteps;

        // ---- staging helpers ----
        auto load_step = [&](int s) {
            const int kbl = s_steps[s];
            const size_t kbyte = (size_t)(seg0 + kbl) * C::ROWB;
#pragma unroll
            for (int i = 0; i < C::NA; ++i) {
                const int q = i * NT + tid;
                const int row = q / C::CPR;
                const int cc = q % C::CPR;
                const int grow = m0 + row;
                if (grow < g.M) {
                    ra[i] = ldg16(A + (size_t)grow * g.K * E::ESZ + kbyte + cc * 16);
                } else {
                    ra[i] = make_uint4(0, 0, 0, 0);
                }
            }
            if constexpr (E::ESZ == 2 && TRANS == 0) {
                // unit = (k pair, 8 columns): two 16-byte rows
#pragma unroll
                for (int i = 0; i < C::NBC / 2; ++i) {
                    const int u = i * NT + tid;
                    const int nl = u / 64;
                    const int w = u % 64;
                    const int b = s_tbl[kbl * NB + nl];
                    if (b >= 0) {
                        const unsigned char* p = D + (size_t)b * 2048 + (w >> 2) * 128 + (w & 3) * 16;
                        rb[2 * i] = ldg16(p);
                        rb[2 * i + 1] = ldg16(p + 64);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < C::NBC; ++i) {
                    const int q = i * NT + tid;
                    const int nl = q / C::CPB;
                    const int cc = q % C::CPB;
                    const int b = s_tbl[kbl * NB + nl];
                    if (b >= 0) rb[i] = ldg16(D + (size_t)b * (1024 * E::ESZ) + cc * 16);
                }
            }
        };
        auto store_step = [&](int s, int buf) {
            const int kbl = s_steps[s];
            unsigned char* sa = stage0 + buf * C::STAGE_BYTES;
            unsigned char* sb = sa + C::A_BYTES;
#pragma unroll
            for (int i = 0; i < C::NA; ++i) {
                const int q = i * NT + tid;
                const int row = q / C::CPR;
                const int cc = q % C::CPR;
                *reinterpret_cast<uint4*>(sa + row * C::PITCH + cc * 16) = ra[i];
            }
            if constexpr (E::ESZ == 2 && TRANS == 0) {
#pragma unroll
                for (int i = 0; i < C::NBC / 2; ++i) {
                    const int u = i * NT + tid;
                    const int nl = u / 64;
                    const int w = u % 64;
                    if (s_tbl[kbl * NB + nl] >= 0) {
                        uint4 lo, hi;
                        interleave_bf16_rows(rb[2 * i], rb[2 * i + 1], lo, hi);
                        // words [k/2][n]: row (w>>2) of 32 words, columns 8*(w&3)..+7
                        uint4* d = reinterpret_cast<uint4*>(sb + nl * C::BLK_BYTES + (w >> 2) * 128 + (w & 3) * 32);
                        d[0] = lo;
                        d[1] = hi;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < C::NBC; ++i) {
                    const int q = i * NT + tid;
                    const int nl = q / C::CPB;
                    const int cc = q % C::CPB;
                    if (s_tbl[kbl * NB + nl] >= 0) {
                        unsigned char* d = sb + nl * C::BLK_BYTES;
                        if constexpr (TRANS) {
                            d += (cc / C::CPR) * C::PITCH + (cc % C::CPR) * 16;
                        } else {
                            d += cc * 16;
                        }
                        *reinterpret_cast<uint4*>(d) = rb[i];
                    }
                }
            }
        };
        auto compute_step = [&](int s, int buf) {
            const int kbl = s_steps[s];
            const unsigned char* sa = stage0 + buf * C::STAGE_BYTES;
            const unsigned char* sb = sa + C::A_BYTES;
            int bsel[TN];
            bool any = false;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                bsel[j] = __builtin_amdgcn_readfirstlane(s_tbl[kbl * NB + wn * TN + j]);
                any |= bsel[j] >= 0;
            }
            if (!any) return;
            uint4 fa[TM][NQ];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const unsigned char* p = sa + ((wm * TM + i) * 32 + lrow) * C::PITCH + h * (C::ROWB / 2);
#pragma unroll
                for (int q = 0; q < NQ; ++q) fa[i][q] = *reinterpret_cast<const uint4*>(p + q * 16);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (bsel[j] < 0) continue;
                const unsigned char* pb = sb + (wn * TN + j) * C::BLK_BYTES;
                uint4 fb[NQ];
                if constexpr (TRANS) {
                    const unsigned char* p = pb + lrow * C::PITCH + h * (C::ROWB / 2);
#pragma unroll
                    for (int q = 0; q < NQ; ++q) fb[q] = *reinterpret_cast<const uint4*>(p + q * 16);
                } else if constexpr (E::ESZ == 4) {
                    const uint32_t* p = reinterpret_cast<const uint32_t*>(pb) + (16 * h) * 32 + lrow;
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        fb[q].x = p[(4 * q + 0) * 32];
                        fb[q].y = p[(4 * q + 1) * 32];
                        fb[q].z = p[(4 * q + 2) * 32];
                        fb[q].w = p[(4 * q + 3) * 32];
                    }
                } else {
                    const uint32_t* p = reinterpret_cast<const uint32_t*>(pb) + (8 * h) * 32 + lrow;
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        fb[q].x = p[(4 * q + 0) * 32];
                        fb[q].y = p[(4 * q + 1) * 32];
                        fb[q].z = p[(4 * q + 2) * 32];
                        fb[q].w = p[(4 * q + 3) * 32];
                    }
                }
#pragma unroll
                for (int i = 0; i < TM; ++i) E::mma(acc[i][j], fa[i], fb);
            }
        };

        // ---- the steps, double buffered: loads of step s+1 are in flight while step s computes ----
        if (ns > 0) {
            load_step(0);
            store_step(0, 0);
            __syncthreads();
            for (int s = 0; s < ns; ++s) {
                const bool more = s + 1 < ns;
                if (more) load_step(s + 1);
                compute_step(s, s & 1);
                if (more) store_step(s + 1, (s + 1) & 1);
                __syncthreads();
            }
        }
    }

    // ---- epilogue: row-major store, bias fused ----
    T* out = static_cast<T*>(g.out);
    const T* bias = static_cast<const T*>(g.bias);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int nb = nb0 + wn * TN + j;
        if (nb >= nblk_n) continue;
        const int col = nb * 32 + lrow;
        const float bv = bias ? E::to_f32(bias[col]) : 0.f;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int rbase = m0 + (wm * TM + i) * 32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = rbase + acc_row(v, h);
                if (row < g.M) out[(size_t)row * g.N + col] = E::from_f32(acc[i][j][v] + bv);
            }
        }
    }
}

}  // namespace pbs
