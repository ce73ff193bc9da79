// dense x block-sparse -> dense (forward Y = X.W^T and input gradient dX = dY.W).
//
// One workgroup owns a BM-token x NB-block-column tile of the result (block columns of the
// *result*: block rows of W for the forward, block columns of W for dX).  Its waves split the
// tokens only: every wave holds accumulators for all NB block columns of its TM*32 tokens and
// runs the same sequence of block products, so the waves of a workgroup always have equal work
// however uneven the pattern is.
//
// The workgroup merges the NB sorted block lists of its tile into one stream of entries ordered by
// k-block (LDS tables), and walks it in steps of SK k-blocks.  Per step the BM x 32 dense operand
// panel of each k-block and the packed blocks of the step's entries are copied global -> LDS by
// the DMA path (global_load_lds_dwordx4, no registers): panels into a ring of RS step buffers,
// blocks into a ring of RB block slots, so that several steps of loads are in flight while one is
// consumed.  Each wave waits for its own DMA instructions with an exact s_waitcnt vmcnt(n), then
// one barrier per step publishes the step to all waves.
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
template <typename T, int TRANS, int TM, int NB, int NW, int SK, int RS, int RB>
struct DdsCfg {
    using E = Elem<T>;
    static constexpr int NT = NW * 64;
    static constexpr int BM = NW * TM * 32;
    static constexpr int SEG = 128;                      // k-blocks merged per table build
    static constexpr int ROWB = 32 * E::ESZ;             // bytes of one 32-wide operand row
    static constexpr int CPR = ROWB / 16;                // 16-byte chunks per row (4 or 8)
    static constexpr int RPI = 64 / CPR;                 // rows filled by one DMA instruction (16 or 8)
    static constexpr int PANEL_BYTES = BM * ROWB;        // one k-block of the dense operand
    static constexpr int PANEL_INSTR = PANEL_BYTES / 1024;
    static constexpr int A_PER_WAVE = PANEL_INSTR / NW;  // DMA instructions per wave per k-block
    static constexpr int STEP_BYTES = SK * PANEL_BYTES;
    static constexpr int BLK_BYTES = 1024 * E::ESZ;
    static constexpr int BLK_INSTR = BLK_BYTES / 1024;   // DMA instructions per packed block (2 or 4)
    static constexpr int A_RING_BYTES = RS * STEP_BYTES;
    static constexpr int B_RING_BYTES = RB * BLK_BYTES;
    // tables: s_tbl[SEG][NB], s_ent[SEG*NB], s_kb[SEG], s_kmask[SEG], s_cum[SEG+1], s_ptr[NB+1], misc[4]
    static constexpr int TBL_INTS = 2 * SEG * NB + 3 * SEG + 1 + NB + 1 + 4;
    static constexpr int LDS_BYTES = A_RING_BYTES + B_RING_BYTES + TBL_INTS * 4;
    static_assert(PANEL_INSTR % NW == 0, "panel DMA must divide evenly over the waves");
    static_assert(RS >= 2, "need at least two step buffers");
    static_assert(RB >= SK * NB, "the block ring must hold one full step");
    static_assert(NB <= 16, "entries keep the block column in 4 bits");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// chunk swizzle of a row: bf16 rows have 4 chunks, fp32 rows 8
template <int CPR>
static __device__ __forceinline__ int swz(int r) {
    return CPR == 4 ? ((r >> 2) & 3) : ((r >> 1) & 7);
}

// one DMA instruction: every lane copies 16 bytes from its global address to LDS chunk (lds_base/16 + lane)
static __device__ __forceinline__ void dma16(unsigned lds_base_uniform, const void* gptr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\t"
                 :
                 : "s"(lds_base_uniform), "v"(gptr)
                 : "memory");
}

// wait until at most n (wave-uniform) of this wave's DMA loads are outstanding, make this wave's
// LDS accesses complete, and meet the other waves.  Loads retire in order, so a smaller n than
// necessary is only slower, never wrong.
static __device__ __forceinline__ void wait_dma_and_barrier(int n) {
#define PBS_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ") lgkmcnt(0)\n\ts_barrier" ::: "memory"); break;
    switch (n) {
        PBS_W(0) PBS_W(1) PBS_W(2) PBS_W(3) PBS_W(4) PBS_W(5) PBS_W(6) PBS_W(7) PBS_W(8)
        PBS_W(9) PBS_W(10) PBS_W(11) PBS_W(12) PBS_W(13) PBS_W(14) PBS_W(15) PBS_W(16)
        PBS_W(17) PBS_W(18) PBS_W(19) PBS_W(20) PBS_W(21) PBS_W(22) PBS_W(23) PBS_W(24)
        PBS_W(25) PBS_W(26) PBS_W(27) PBS_W(28) PBS_W(29) PBS_W(30) PBS_W(31) PBS_W(32)
        PBS_W(33) PBS_W(34) PBS_W(35) PBS_W(36) PBS_W(37) PBS_W(38) PBS_W(39) PBS_W(40)
        default: asm volatile("s_waitcnt vmcnt(40) lgkmcnt(0)\n\ts_barrier" ::: "memory"); break;
    }
#undef PBS_W
}
static __device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <typename T, int TRANS, int TM, int NB, int NW, int SK, int RS, int RB>
__global__ __launch_bounds__(NW * 64) void dds_kernel(DdsArgs g) {
    using C = DdsCfg<T, TRANS, TM, NB, NW, SK, RS, RB>;
    using E = typename C::E;
    constexpr int NT = C::NT, SEG = C::SEG, NQ = E::NQ, CPR = C::CPR;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    unsigned char* const a_ring = smem;
    unsigned char* const b_ring = smem + C::A_RING_BYTES;
    int* s_tbl = reinterpret_cast<int*>(smem + C::A_RING_BYTES + C::B_RING_BYTES);  // [SEG][NB] block or -1
    int* s_ent = s_tbl + SEG * NB;   // entries in (k-block, block column) order: (data block << 4) | column
    int* s_kb = s_ent + SEG * NB;    // [SEG] k-block (local to the segment) of each present k-block
    int* s_kmask = s_kb + SEG;       // [SEG] block columns present in each present k-block
    int* s_cum = s_kmask + SEG;      // [SEG+1] entries before each present k-block
    int* s_ptr = s_cum + SEG + 1;    // [NB+1]
    int* s_misc = s_ptr + NB + 1;    // [0] = number of present k-blocks
    const unsigned lds_a = (unsigned)(uintptr_t)a_ring;
    const unsigned lds_b = (unsigned)(uintptr_t)b_ring;

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
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane & 31;
    const int h = lane >> 5;

    const unsigned char* A = static_cast<const unsigned char*>(g.a);
    const unsigned char* D = static_cast<const unsigned char*>(g.data);

    f32x16 acc[TM][NB];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    if (tid <= NB) {
        int nb = nb0 + tid;
        s_ptr[tid] = g.ptr[nb < nblk_n ? nb : nblk_n];
    }
    __syncthreads();
    const int e_begin = s_ptr[0];
    const int e_end = s_ptr[NB];

    // ---- per-lane constants of the DMA address patterns ----
    // panel: this wave fills instructions wave*A_PER_WAVE + i of every k-block; lane p of instruction q
    // serves row q*RPI + p/CPR and physical chunk p%CPR, i.e. logical chunk (p%CPR) ^ swz(row)
    const unsigned char* a_src[C::A_PER_WAVE];
#pragma unroll
    for (int i = 0; i < C::A_PER_WAVE; ++i) {
        const int q = wave * C::A_PER_WAVE + i;
        const int row = q * C::RPI + lane / CPR;
        const int chunk = (lane % CPR) ^ swz<CPR>(row);
        int grow = m0 + row;
        if (grow >= g.M) grow = g.M - 1;   // rows past the end re-read the last row; their results are never stored
        a_src[i] = A + (size_t)grow * g.K * E::ESZ + chunk * 16;
    }
    // packed block: instruction q of a block; forward keeps the block as stored, dX swizzles rows
    int b_off[C::BLK_INSTR];
#pragma unroll
    for (int q = 0; q < C::BLK_INSTR; ++q) {
        if constexpr (TRANS) {
            const int row = q * C::RPI + lane / CPR;
            b_off[q] = row * C::ROWB + ((lane % CPR) ^ swz<CPR>(row)) * 16;
        } else {
            b_off[q] = q * 1024 + lane * 16;
        }
    }
    // per-lane offsets of the fragment reads
    int a_frag_off[TM][NQ];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = (wave * TM + i) * 32 + lrow;
#pragma unroll
        for (int q = 0; q < NQ; ++q) a_frag_off[i][q] = row * C::ROWB + (((h * NQ + q) ^ swz<CPR>(row)) * 16);
    }
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

    // number of block-DMA issues of this wave among entries [0, x): entry e is copied by wave e % NW
    auto my_blocks_before = [&](int x) -> int { return (x + NW - 1 - wave) / NW; };

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
            // wave 0 compacts: present k-blocks, entries before each, and the entry stream
            int nk = 0, ne = 0;
            for (int base = 0; base < SEG; base += 64) {
                const int kbl = base + lane;
                int present = 0;
#pragma unroll
                for (int j = 0; j < NB; ++j) present |= (s_tbl[kbl * NB + j] >= 0) ? (1 << j) : 0;
                const int cnt = __popc(present);
                const unsigned long long m = __ballot(cnt != 0);
                // exclusive scan of cnt over the 64 lanes
                int incl = cnt;
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) {
                    const int o = __shfl_up(incl, d, 64);
                    if (lane >= d) incl += o;
                }
                const int total = __shfl(incl, 63, 64);
                if (cnt) {
                    const int pos = nk + __popcll(m & ((1ull << lane) - 1ull));
                    int e = ne + incl - cnt;
                    s_kb[pos] = kbl;
                    s_kmask[pos] = present;
                    s_cum[pos] = e;
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const int b = s_tbl[kbl * NB + j];
                        if (b >= 0) s_ent[e++] = (b << 4) | j;
                    }
                }
                nk += __popcll(m);
                ne += total;
            }
            if (lane == 0) {
                s_cum[nk] = ne;
                s_misc[0] = nk;
            }
        }
        __syncthreads();
        const int nk = s_misc[0];
        const int ns = (nk + SK - 1) / SK;

        // first present-k-block index after step s, and entries before it
        auto kend = [&](int s) -> int { const int i = (s + 1) * SK; return i < nk ? i : nk; };
        auto cum = [&](int i) -> int { return __builtin_amdgcn_readfirstlane(s_cum[i]); };
        // DMA instructions this wave has issued once steps 0..s are issued
        auto issued_through = [&](int s) -> int {
            const int i = kend(s);
            return C::A_PER_WAVE * i + C::BLK_INSTR * my_blocks_before(cum(i));
        };
        auto issue_step = [&](int s) {
            const int i0 = s * SK, i1 = kend(s);
            const unsigned stage = lds_a + (s % RS) * C::STEP_BYTES;
            for (int i = i0; i < i1; ++i) {
                const int kbl = __builtin_amdgcn_readfirstlane(s_kb[i]);
                const size_t kbyte = (size_t)(seg0 + kbl) * C::ROWB;
                const unsigned dst = stage + (i - i0) * C::PANEL_BYTES + wave * C::A_PER_WAVE * 1024;
#pragma unroll
                for (int q = 0; q < C::A_PER_WAVE; ++q) dma16(dst + q * 1024, a_src[q] + kbyte);
            }
            const int e0 = cum(i0), e1 = cum(i1);
            int e = e0 + ((wave - e0) % NW + NW) % NW;   // first entry >= e0 with e % NW == wave
            for (; e < e1; e += NW) {
                const int b = __builtin_amdgcn_readfirstlane(s_ent[e]) >> 4;
                const unsigned char* src = D + (size_t)b * C::BLK_BYTES;
                const unsigned dst = lds_b + (e % RB) * C::BLK_BYTES;
#pragma unroll
                for (int q = 0; q < C::BLK_INSTR; ++q) dma16(dst + q * 1024, src + b_off[q]);
            }
        };
        // step t may be issued while step s is the oldest unconsumed one if its panel buffer and its
        // block slots are free
        auto can_issue = [&](int t, int s) -> bool {
            return t < ns && t <= s + RS - 1 && cum(kend(t)) - cum(s * SK) <= RB;
        };

        auto load_a = [&](uint4 (&fa)[TM][NQ], const unsigned char* panel) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int q = 0; q < NQ; ++q) fa[i][q] = *reinterpret_cast<const uint4*>(panel + a_frag_off[i][q]);
        };
        auto load_b = [&](uint4 (&fb)[NQ], const unsigned char* pb) {
            if constexpr (TRANS) {
                const unsigned char* p = pb + b_frag_off;
                const int sw = swz<CPR>(lrow);
#pragma unroll
                for (int q = 0; q < NQ; ++q) fb[q] = *reinterpret_cast<const uint4*>(p + (((h * NQ + q) ^ sw) * 16));
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
        auto compute_step = [&](int s) {
            const int i0 = s * SK, i1 = kend(s);
            const unsigned char* stage = a_ring + (s % RS) * C::STEP_BYTES;
            int e = cum(i0);
            uint4 fb[NQ];
            load_b(fb, b_ring + (e % RB) * C::BLK_BYTES);
            for (int i = i0; i < i1; ++i) {
                const int mask = __builtin_amdgcn_readfirstlane(s_kmask[i]);
                uint4 fa[TM][NQ];
                load_a(fa, stage + (i - i0) * C::PANEL_BYTES);
                // block columns in order; the accumulator index stays static, the branches are uniform.
                // The next entry's block fragment is always fetched before the products of this one are
                // issued (past the last entry of the step that is an unused slot), so the read latency
                // hides behind the matrix-core work without any path-dependent wait.
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    if ((mask >> j) & 1) {
                        uint4 fb_next[NQ];
                        ++e;
                        load_b(fb_next, b_ring + (e % RB) * C::BLK_BYTES);
#pragma unroll
                        for (int t = 0; t < TM; ++t) E::mma(acc[t][j], fa[t], fb);
#pragma unroll
                        for (int q = 0; q < NQ; ++q) fb[q] = fb_next[q];
                    }
                }
            }
        };

        // ---- the steps ----
        if (ns > 0) {
            int next = 0;
#ifndef PBS_EXP_NO_DMA
            while (can_issue(next, 0)) issue_step(next++);
#else
            next = ns;
#endif
            for (int s = 0; s < ns; ++s) {
                if (next <= s) {
                    // the block ring could not take step s while step s-1 was in use
                    lds_barrier();
                    issue_step(s);
                    next = s + 1;
                }
                wait_dma_and_barrier(issued_through(next - 1) - issued_through(s));
                // every wave is past step s-1 now: its buffers can be refilled
#ifndef PBS_EXP_NO_DMA
                if (s > 0)
                    while (can_issue(next, s)) issue_step(next++);
#endif
#ifndef PBS_EXP_NO_COMPUTE
                compute_step(s);
#endif
            }
            // the tables and the rings are rewritten next: wait for the last reads
            lds_barrier();
        }
    }

#ifdef PBS_EXP_NO_EPILOGUE
    if (g.M > 0) return;
#endif
    // ---- epilogue: row-major store, bias fused ----
    T* out = static_cast<T*>(g.out);
    const T* bias = static_cast<const T*>(g.bias);
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int nb = nb0 + j;
        if (nb < nblk_n) {
            const int col = nb * 32 + lrow;
            const float bv = bias ? E::to_f32(bias[col]) : 0.f;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int rbase = m0 + (wave * TM + i) * 32;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = rbase + acc_row(v, h);
                    if (row < g.M) out[(size_t)row * g.N + col] = E::from_f32(acc[i][j][v] + bv);
                }
            }
        }
    }
}

}  // namespace pbs
