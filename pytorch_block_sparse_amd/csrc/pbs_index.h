// Device-side build of the five int32 index arrays of a block mask.
//
// One workgroup of 1024 threads does the whole job (the grids are at most a few hundred thousand
// positions and this runs only when a pattern is created or changed).  Pass 1 walks the mask in
// row-major order: an exclusive scan of per-thread counts gives every nonzero its rank i, hence
// cols_a[i] = (col, block_ptr[i]), the row starts and blocks[block_ptr[i]] = (col, row).  Pass 2
// walks it in column-major order for rows_b / col_start_ends_b and finds each nonzero's data
// block by a binary search of its column in the (sorted) CSR row written by pass 1.
#pragma once
#include "pbs_common.h"

namespace pbs {

constexpr int INDEX_THREADS = 1024;

// exclusive scan of one int per thread over the workgroup; *total gets the sum
static __device__ int block_exclusive_scan(int v, int* s_wave /*[17]*/, int* total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
    }
    __syncthreads();   // s_wave may still be read from a previous scan
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int w = 0; w < INDEX_THREADS / 64; ++w) {
            const int c = s_wave[w];
            s_wave[w] = run;
            run += c;
        }
        s_wave[16] = run;
    }
    __syncthreads();
    *total = s_wave[16];
    return s_wave[wave] + incl - v;
}

__global__ __launch_bounds__(INDEX_THREADS) void build_indices_kernel(
    const uint8_t* __restrict__ mask, const int64_t* __restrict__ block_ptr, int X, int Y, int nnz,
    int32_t* cols_a, int32_t* row_ptr, int32_t* rows_b, int32_t* col_ptr, int32_t* blocks, int32_t* status) {
    __shared__ int s_wave[17];
    __shared__ int s_err;
    const int tid = threadIdx.x;
    const long long total = (long long)X * Y;
    const long long chunk = (total + INDEX_THREADS - 1) / INDEX_THREADS;
    long long lo = tid * chunk, hi = lo + chunk;
    if (lo > total) lo = total;
    if (hi > total) hi = total;
    if (tid == 0) s_err = 0;

    // ---- pass 1: row-major ----
    int cnt = 0;
    for (long long p = lo; p < hi; ++p) cnt += mask[p] ? 1 : 0;
    int counted;
    int rank = block_exclusive_scan(cnt, s_wave, &counted);
    if (counted != nnz) {
        if (tid == 0) {
            status[0] = counted;
            status[1] = 1;
        }
        return;
    }
    for (long long p = lo; p < hi; ++p) {
        const int r = (int)(p / Y), c = (int)(p % Y);
        if (c == 0) row_ptr[r] = rank;
        if (mask[p]) {
            long long bp = block_ptr ? block_ptr[rank] : rank;
            if (bp < 0 || bp >= nnz) {
                s_err = 2;
                bp = -1;
            }
            cols_a[2 * rank] = c;
            cols_a[2 * rank + 1] = (int)bp;
            if (bp >= 0) {
                blocks[2 * bp] = c;
                blocks[2 * bp + 1] = r;
            }
            ++rank;
        }
    }
    if (tid == 0) row_ptr[X] = nnz;
    __threadfence();
    __syncthreads();

    // ---- pass 2: column-major ----
    cnt = 0;
    for (long long q = lo; q < hi; ++q) {
        const int c = (int)(q / X), r = (int)(q % X);
        cnt += mask[(long long)r * Y + c] ? 1 : 0;
    }
    rank = block_exclusive_scan(cnt, s_wave, &counted);
    for (long long q = lo; q < hi; ++q) {
        const int c = (int)(q / X), r = (int)(q % X);
        if (r == 0) col_ptr[c] = rank;
        if (mask[(long long)r * Y + c]) {
            int l = row_ptr[r], u = row_ptr[r + 1];
            while (l < u) {
                const int mid = (l + u) >> 1;
                if (cols_a[2 * mid] < c) l = mid + 1; else u = mid;
            }
            rows_b[2 * rank] = r;
            rows_b[2 * rank + 1] = cols_a[2 * l + 1];
            ++rank;
        }
    }
    if (tid == 0) col_ptr[Y] = nnz;
    __syncthreads();
    if (tid == 0) {
        status[0] = nnz;
        status[1] = s_err;
    }
}

// ---- the CSR pair of a pattern given as the reference's `blocks` list ----
// blocks[2 b] = block column, blocks[2 b + 1] = block row of data block b, in any order.  owner[p] = data block
// at row-major position p of the X x Y grid, or -1; then one row-major sweep of owner writes cols_a (sorted by
// row, then column) and the row starts.  A position listed twice keeps one of its data blocks (the other gets no
// result); entries outside the grid are skipped.
__global__ __launch_bounds__(256) void blocks_owner_clear_kernel(int* owner, long long total) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) owner[i] = -1;
}
__global__ __launch_bounds__(256) void blocks_owner_kernel(const int32_t* __restrict__ blocks, int nnz, int X, int Y, int* owner) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= nnz) return;
    const int c = blocks[2 * b], r = blocks[2 * b + 1];
    if (c >= 0 && c < Y && r >= 0 && r < X) owner[(long long)r * Y + c] = b;
}
__global__ __launch_bounds__(INDEX_THREADS) void csr_from_owner_kernel(const int* __restrict__ owner, int X, int Y,
                                                                       int32_t* cols_a, int32_t* row_ptr) {
    __shared__ int s_wave[17];
    const int tid = threadIdx.x;
    const long long total = (long long)X * Y;
    const long long chunk = (total + INDEX_THREADS - 1) / INDEX_THREADS;
    long long lo = tid * chunk, hi = lo + chunk;
    if (lo > total) lo = total;
    if (hi > total) hi = total;
    int cnt = 0;
    for (long long p = lo; p < hi; ++p) cnt += owner[p] >= 0 ? 1 : 0;
    int counted;
    int rank = block_exclusive_scan(cnt, s_wave, &counted);
    for (long long p = lo; p < hi; ++p) {
        const int r = (int)(p / Y), c = (int)(p % Y);
        if (c == 0) row_ptr[r] = rank;
        const int b = owner[p];
        if (b >= 0) {
            cols_a[2 * rank] = c;
            cols_a[2 * rank + 1] = b;
            ++rank;
        }
    }
    if (tid == 0) row_ptr[X] = counted;
}

// out[c][r] = in[r][c] for a rows x cols matrix of 2- or 4-byte elements (tiles of 32 x 32 through LDS)
template <typename U>
__global__ __launch_bounds__(256) void transpose_dense_kernel(const U* __restrict__ in, U* __restrict__ out, long long rows,
                                                              long long cols) {
    __shared__ U s[32][33];
    const long long r0 = (long long)blockIdx.y * 32, c0 = (long long)blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const long long r = r0 + ty + i, c = c0 + tx;
        if (r < rows && c < cols) s[ty + i][tx] = in[r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const long long c = c0 + ty + i, r = r0 + tx;
        if (r < rows && c < cols) out[c * rows + r] = s[tx][ty + i];
    }
}

}  // namespace pbs
