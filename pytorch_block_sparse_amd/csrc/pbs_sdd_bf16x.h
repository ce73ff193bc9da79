// bf16 weight gradient on the sparse support without barriers in the token loop.
//
//   out[32b + j][i] = sum_t G[t][32r + i] * X[t][32c + j]   for every data block b at (r, c).
//
// Same decomposition as sdd_bf16_kernel (pbs_sdd_bf16.h): one workgroup of 8 waves owns a 16 x 16 rectangle of
// block positions and one slice of the tokens, the blocks present are dealt to the waves in equal runs, the
// operand panels of a chunk of tokens go global -> LDS by DMA and both matrix operands are gathered with
// transposing reads.  What differs is who copies and when.  There a chunk is 32 tokens in one of two buffers, every
// wave copies its share of the next chunk between its own block products, and a barrier ends the chunk: a wave's
// copy instructions hold it up until the texture path has taken them, its fragment reads and its matrix
// instructions follow, and the three phases add up.  Here a chunk is 16 tokens in one of four buffers, there is no
// barrier, and a chunk is copied whole by one wave: after every chunk of its own a wave looks at the progress
// words, and if a buffer is free (every wave has left the chunk it held) and nobody has claimed the next chunk yet,
// it claims it with a compare-and-swap and copies it, while the other seven go on multiplying.  The wave that has
// copied is then the last to finish its chunk, so the next claim falls to another one: the copying rotates by
// itself, and the texture path, the LDS and the matrix cores work at the same time.
//
// Progress words in LDS: done[w] = the chunk wave w needs next (it has finished reading every earlier one),
// landed[s] = buffer s holds chunk landed[s] - 1 (written by the copying wave after it has waited for its own
// loads: s_waitcnt vmcnt(0); the multiplying waves issue no vector-memory instructions in the loop, so that
// counter is the copier's alone), next = the first chunk nobody has copied yet.  Chunk c may overwrite buffer
// c % 4 once min done[] > c - 4.  Every wait sleeps between polls and is bounded; one that runs out (a broken
// protocol) is counted and turns the results into NaN.
//
// LDS layout of a buffer: G panel then X panel, 16 token rows each, a row pitch of 1024 + 64 bytes: the
// transposing reads take 32 bytes from each of 4 consecutive token rows per 16 lanes, and the 64 extra bytes
// put those on different banks (the barrier kernel swizzles the rows instead, which a wave that copies all
// rows of a chunk would have to undo per row).
#pragma once
#include "pbs_common.h"
#include "pbs_sdd.h"
#include "pbs_sdd_bf16.h"

namespace pbs {

template <int QW>
struct SddBf16xCfg {
    static constexpr int SR = 16, SC = 16, NW = 8, NT = NW * 64;
    static constexpr int TC = 16;                          // tokens per chunk: one matrix step of 16
    static constexpr int NS = 4;                           // chunk buffers
    static constexpr int PITCH = 1024 + 64;                // bytes from one token row of a panel to the next
    static constexpr int PANEL_BYTES = TC * PITCH;
    static constexpr int STAGE_BYTES = 2 * PANEL_BYTES;    // G panel, then X panel
    static constexpr int RING_BYTES = NS * STAGE_BYTES;
    static constexpr int LIST_MAX = SR * SC;
    static constexpr int QMAX = QW * NW;
    static constexpr int LISTS_BYTES = LIST_MAX * 4 + LIST_MAX * 2 + 256;   // s_blk, s_pos, s_rowoff + s_rowid + s_gu
    static constexpr int WORDS_OFF = RING_BYTES + LISTS_BYTES;              // done[8], landed[4], next, fail
    static constexpr int LDS_BYTES = WORDS_OFF + 64;
    static constexpr int SPIN_LIMIT = 1 << 18;
    static_assert((2 * SR + SC / 2 + 4) * 4 <= 256, "the small tables fit their 256 bytes");
    static_assert(SDD_BF16_PROLOGUE_BYTES <= RING_BYTES, "the prologue's scratch fits in the chunk buffers");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

template <int QW>
__global__ __launch_bounds__(512) void sdd_bf16x_kernel(SddArgs a) {
    using C = SddBf16xCfg<QW>;
    constexpr int NS = C::NS, SR = C::SR, SC = C::SC, NW = C::NW, TC = C::TC, PITCH = C::PITCH;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    int* s_blk = reinterpret_cast<int*>(smem + C::RING_BYTES);                        // [LIST_MAX] data block
    unsigned short* s_pos = reinterpret_cast<unsigned short*>(s_blk + C::LIST_MAX);  // [LIST_MAX] (rl << 8) | cl
    int* s_rowoff = reinterpret_cast<int*>(s_pos + C::LIST_MAX);                     // [SR + 1]
    int* s_rowid = s_rowoff + SR + 2;   // [SR] block row of W in each place of this rectangle's band, or -1
    int* s_gu = s_rowid + SR;           // [SC / 2] column unit in each place of this rectangle, or -1
    int* const s_done = reinterpret_cast<int*>(smem + C::WORDS_OFF);   // [8]
    int* const s_landed = s_done + NW;                                 // [4]
    int* const s_next = s_landed + NS;
    int* const s_fail = s_next + 1;
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

    const int nblk_c = a.K / 32;
    sdd_bf16_prologue<C::NT>(a, tile, smem, s_blk, s_pos, s_rowoff, s_rowid, s_gu);
    const int nq = __builtin_amdgcn_readfirstlane(s_rowoff[SR]);
    if (nq == 0) return;

    const int t_begin = sp * a.tokens_per_split;
    int t_end = t_begin + a.tokens_per_split;
    if (t_end > a.M) t_end = a.M;
    const int nchunks = t_begin < t_end ? (t_end - t_begin + TC - 1) / TC : 0;

    // ---- DMA address pattern: one instruction per token row and panel; lane l fetches the row's 16-byte chunk l ----
    const unsigned char* G = static_cast<const unsigned char*>(a.g);
    const unsigned char* X = static_cast<const unsigned char*>(a.x);
    // G: the 64 bytes of place l / 4 of the band come from that place's block row (a place without a row fetches some
    // valid address; nothing reads it)
    const int g_rid = s_rowid[lane >> 2];
    const unsigned g_voff = (g_rid >= 0 && g_rid < a.N / 32) ? (unsigned)(g_rid * 64 + (lane & 3) * 16) : 0u;
    // X: the 64 bytes of place l / 4 come from that place's block column (two adjacent columns per unit)
    const int x_unit = s_gu[lane >> 3];
    const int x_cid = x_unit >= 0 ? x_unit * 2 + ((lane >> 2) & 1) : -1;
    const unsigned x_voff = (x_cid >= 0 && x_cid < nblk_c) ? (unsigned)(x_cid * 64 + (lane & 3) * 16) : 0u;
    const size_t g_row_bytes = (size_t)a.N * 2, x_row_bytes = (size_t)a.K * 2;

    // all rows of chunk c into buffer c % NS, then (after this wave's loads have landed) the chunk's number on landed[]
    auto copy_chunk = [&](int c) __attribute__((always_inline)) {
        c = __builtin_amdgcn_readfirstlane(c);
        const unsigned stage = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(c & (NS - 1)) * C::STAGE_BYTES);
        const int t0 = t_begin + c * TC;
        const unsigned char* pg = uniform_ptr(G + (size_t)t0 * g_row_bytes);
        const unsigned char* px = uniform_ptr(X + (size_t)t0 * x_row_bytes);
        int lc = lane;
        asm volatile("" : "+v"(lc));
#pragma unroll 1
        for (int r = 0; r < TC; ++r) {
            const unsigned dst = __builtin_amdgcn_readfirstlane(stage + (unsigned)r * PITCH);
            if (t0 + r < t_end) {
                dma16(dst, pg, g_voff);
                dma16(dst + C::PANEL_BYTES, px, x_voff);
            } else {
                // tokens past the end contribute nothing
                unsigned char* p = smem + (dst - lds0) + lc * 16;
                *reinterpret_cast<uint4*>(p) = make_uint4(0, 0, 0, 0);
                *reinterpret_cast<uint4*>(p + C::PANEL_BYTES) = make_uint4(0, 0, 0, 0);
            }
            pg = uniform_ptr(pg + g_row_bytes);
            px = uniform_ptr(px + x_row_bytes);
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        if (lane == 0) lds_poke(s_landed + (c & (NS - 1)), c + 1);
    };

    // ---- progress words ----
    bool gave_up = false;
    int md = 0;   // last minimum of done[] seen (it only grows)
    // all words in one read: lanes 0..7 done[lane], lane 8 the landed word of chunk c's buffer, the others next
    auto poll_all = [&](int c) __attribute__((always_inline)) -> int {
        int l = lane;
        asm volatile("" : "+v"(l));
        const int idx = l < NW ? l : (l == NW ? NW + (c & (NS - 1)) : NW + NS);
        return lds_peek(s_done + idx);
    };
    // Copy every chunk whose buffer is free and that this wave manages to claim; v = what poll_all has read.
    auto copy_free_chunks = [&](int v) __attribute__((always_inline)) {
        int nc = __builtin_amdgcn_readlane(v, NW + 1);
        int m = v;
#define PBS_MIN_SHR(SH)                                                                  \
    {                                                                                    \
        const int m2 = __builtin_amdgcn_update_dpp(m, m, 0x110 + SH, 0xf, 0xf, false);   \
        m = m2 < m ? m2 : m;                                                             \
    }
        PBS_MIN_SHR(1) PBS_MIN_SHR(2) PBS_MIN_SHR(4)
#undef PBS_MIN_SHR
        const int dmin = __builtin_amdgcn_readlane(m, NW - 1);   // minimum of lanes 0..7
        md = dmin > md ? dmin : md;
        while (nc < nchunks && nc - NS < md) {
            int expected = nc;
            if (lane == 0)
                __hip_atomic_compare_exchange_strong((lds_int*)s_next, &expected, nc + 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_WORKGROUP);
            expected = __builtin_amdgcn_readfirstlane(expected);   // what the word held: nc if the claim is this wave's
            if (expected == nc) {
                copy_chunk(nc);
                ++nc;
            } else {
                nc = expected;
            }
        }
    };
    // wait until chunk c is there, copying what is free meanwhile
    auto wait_chunk = [&](int c) __attribute__((always_inline)) {
        bool here = false;
        for (int spin = 0; spin < C::SPIN_LIMIT; ++spin) {
            const int v = poll_all(c);
            here = __builtin_amdgcn_readlane(v, NW) > c;
            if (here) break;
            copy_free_chunks(v);
            if ((spin & 1023) == 1023 && __builtin_amdgcn_readfirstlane(lds_peek(s_fail)) != 0) break;
            __builtin_amdgcn_s_sleep(2);
        }
        if (!here) {
            gave_up = true;
            if (lane == 0) lds_poke(s_fail, 1);
            count_protocol_failure();
        }
    };

    // ---- per-lane part of the fragment addresses ----
    // transposing read: within 16 lanes, lane s addresses 4 consecutive features of token row s/4 and
    // receives, for its own feature, the 4 token rows as 4 consecutive k.  Lane l serves feature
    // (l & 31) of the block; lane half h serves tokens 8h..8h+7 of the 16-token matrix step.
    const int l16 = lane & 15;
    const int trow = 8 * h + (l16 >> 2);                              // + 4 for the second read
    const int cb = 2 * ((lane >> 4) & 1) + ((l16 & 3) >> 1);          // 16-byte chunk inside the block's 64 bytes
    const int lane_const = trow * PITCH + (l16 & 1) * 8;
    auto frag_off = [&](int blk16) -> int { return lane_const + (blk16 * 4 + cb) * 16; };

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
            a_off[q] = C::PANEL_BYTES + frag_off(pos & 15);
            b_off[q] = frag_off((pos >> 8) & 15);
            blk_of[q] = q < w_n ? __builtin_amdgcn_readfirstlane(s_blk[w_lo + q]) : -1;
        }

        f32x16 acc[QW];
#pragma unroll
        for (int q = 0; q < QW; ++q)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[q][v] = 0.f;

        // the progress words start from zero in every pass; nothing of the previous pass is in flight (a wave that
        // copies waits for its loads before it goes on) and every wave has left the last chunk's buffer
        __syncthreads();
        if (tid < NW + NS + 2) s_done[tid] = 0;
        md = 0;
        __syncthreads();

        auto load_frag = [&](uint4& f, const unsigned char* p) __attribute__((always_inline)) {
            const uint2 lo = tr16_b64(p);
            const uint2 hi = tr16_b64(p + 4 * PITCH);
            f = make_uint4(lo.x, lo.y, hi.x, hi.y);
        };
        for (int ci = 0; ci < nchunks; ++ci) {
            if (__builtin_amdgcn_readfirstlane(lds_peek(s_landed + (ci & (NS - 1)))) <= ci && !gave_up) wait_chunk(ci);
            // (the compiler does not see who writes the buffers: no read of them may move above the check)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            const unsigned char* stage = smem + (ci & (NS - 1)) * C::STAGE_BYTES;
            // the fragments of block q + 1 are fetched before the product of block q is issued
            uint4 fa[2], fb[2];
            if (w_n > 0) {
                load_frag(fb[0], stage + b_off[0]);
                load_frag(fa[0], stage + a_off[0]);
            }
#pragma unroll
            for (int q = 0; q < QW; ++q) {
                if (q < w_n) {
                    uint4& fa_c = fa[q & 1];
                    uint4& fb_c = fb[q & 1];
                    uint4& fa_n = fa[(q & 1) ^ 1];
                    uint4& fb_n = fb[(q & 1) ^ 1];
                    if (q + 1 < QW && q + 1 < w_n) {
                        load_frag(fa_n, stage + a_off[q + 1]);
                        if (rl_of[q + 1] != rl_of[q]) load_frag(fb_n, stage + b_off[q + 1]);
                        else fb_n = fb_c;
                    }
                    acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa_c), __builtin_bit_cast(bf16x8, fb_c),
                                                                     acc[q], 0, 0, 0);
                }
            }
            // this wave has read everything it needs of chunk ci (the matrix instructions above have their operands)
            asm volatile("" ::: "memory");
            if (lane == 0) lds_poke(s_done + wave, ci + 1);
            // and looks whether a buffer has become free for a chunk nobody has copied yet
            if (!gave_up) copy_free_chunks(poll_all(ci + 1));
        }
        if (lane == 0) lds_poke(s_done + wave, 0x7fffffff);

        // ---- store: result row j (X feature), column i (G feature) ----
        const bool failed = gave_up || __builtin_amdgcn_readfirstlane(lds_peek(s_fail)) != 0;
#pragma unroll
        for (int q = 0; q < QW; ++q) {
            if (q < w_n && blk_of[q] >= 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const size_t o = (size_t)blk_of[q] * 1024 + acc_row(v, h) * 32 + lrow;
                    const float r = failed ? __builtin_nanf("") : acc[q][v];
                    if (part) part[o] = r;
                    else out[o] = Elem<bf16_t>::from_f32(r);
                }
            }
        }
    }
}

}  // namespace pbs
