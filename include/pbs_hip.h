/*
 * pbs_hip.h -- C ABI of libpbs_hip.so, the MI355X (gfx950) block-sparse matmul engine.
 *
 * Plain C: raw device pointers, sizes and a hipStream_t passed as void*.  No torch
 * types.  All pointers are caller-owned device memory; the library keeps nothing
 * after a call returns, so calls on different streams or from different host threads
 * do not interfere.  Its only device state of its own: the scratch array of the entry
 * point that allocates nothing (see there) and one diagnostic counter.
 *
 * Every entry point returns an int: 0 on success, a positive hipError_t when the HIP
 * runtime reported an error, a negative PBS_ERR_* when an argument was rejected
 * before anything was launched.  pbs_error_string() turns either into text.
 *
 * Data conventions (those of the reference's BlockSparseMatrix, block_sparse.py):
 *   - the weight W is [out_features, in_features], tiled in 32x32 blocks; X = out/32
 *     block rows, Y = in/32 block columns, nnz nonzero blocks;
 *   - packed data is [nnz*32, 32] row-major; data block b holds its W block
 *     transposed: data[32b + j][i] = W[32r + i][32c + j]      (block_sparse.py:326-331)
 *   - row_start_ends_a [X+1], cols_a [nnz][2] = (block col, data block)   CSR
 *   - col_start_ends_b [Y+1], rows_b [nnz][2] = (block row, data block)   CSC
 *   - blocks [nnz][2] = (block col, block row) of data block b         (:138-141)
 *   - dense operands are row-major and contiguous; dense results are row-major.
 */
#ifndef PBS_HIP_H
#define PBS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PBS_ABI_VERSION 4
#define PBS_BLOCK 32

/* element type of dense operands, packed data and results (accumulation is fp32) */
#define PBS_DTYPE_F32 0
#define PBS_DTYPE_BF16 1

#define PBS_OK 0
#define PBS_ERR_NULL_POINTER (-1)
#define PBS_ERR_BAD_SHAPE (-2)     /* negative size or a feature dim not a multiple of 32 */
#define PBS_ERR_BAD_DTYPE (-3)
#define PBS_ERR_MISALIGNED (-4)    /* a dense/data pointer is not 16-byte aligned */
#define PBS_ERR_WORKSPACE (-5)     /* workspace/plan buffer missing, misaligned or too small */
#define PBS_ERR_TOO_LARGE (-6)     /* a size exceeds what the kernels index with */
#define PBS_ERR_SCRATCH (-7)       /* more scratch needed than the built-in buffer of the no-allocation entry point */

int pbs_abi_version(void);
const char* pbs_error_string(int code);

/*
 * Index arrays of a block mask, built on the device, bit-exact with the reference's
 * BlockSparseMatrixBase.build_indices (block_sparse.py:125-153, helper :85-123).
 *
 *   mask       [X*Y] bytes, row-major, nonzero = block present
 *   block_ptr  NULL, or [nnz] int64: data-block id of the i-th nonzero in row-major
 *              order (the "recycled blocks" path used by block_replace, :210-219)
 *   nnz        the number of blocks the caller allocated outputs for
 *   status     [2] int32 device words: status[0] = number of nonzeros counted in mask,
 *              status[1] = 0 if ok, 1 if the count differs from nnz (nothing else is
 *              written then), 2 if a block_ptr entry is outside [0, nnz)
 */
int pbs_build_indices(const uint8_t* mask, const int64_t* block_ptr, int X, int Y, int nnz,
                      int32_t* cols_a, int32_t* row_start_ends_a,
                      int32_t* rows_b, int32_t* col_start_ends_b,
                      int32_t* blocks, int32_t* status, void* stream);

/*
 * Schedule ("plan") of the dense x block-sparse product for one pattern and one direction.
 * It depends only on the index arrays, not on the data: build it when the pattern is created or
 * changed and pass it to every pbs_blocksparse_matmul call of that direction.  It is what the
 * reference's kernel derives again in every thread block from ptr/indices
 * (cutlass/gemm/block_loader_crosswise_prune_dense.h:254-264, :398-444), hoisted out of the hot
 * path: per group of 8 result block columns, the merged list of k-blocks they touch.
 *
 *   transpose = 1 (forward):        ptr = row_start_ends_a, indices = cols_a, n = out, k = in
 *   transpose = 0 (input gradient): ptr = col_start_ends_b, indices = rows_b, n = in,  k = out
 *   plan: 16-byte aligned device buffer of pbs_blocksparse_matmul_plan_bytes(n, k) bytes
 */
size_t pbs_blocksparse_matmul_plan_bytes(int n, int k);
int pbs_blocksparse_matmul_plan(const int32_t* ptr, const int32_t* indices, int n, int k, int nnz,
                                void* plan, size_t plan_bytes, void* stream);

/*
 * dense x block-sparse -> dense.  Replaces blocksparse_matmul_cutlass
 * (native/block_sparse_native.cpp:6-16, launcher native/block_sparse_cutlass_kernel.cu:113-150)
 * as called by BlockSparseMatrixBase.reverse_matmul_ (block_sparse.py:496-578).
 *
 *   transpose = 1 : out[tokens, n] = a[tokens, k] . W^T   n = out_features, k = in_features  (:518-521)
 *   transpose = 0 : out[tokens, n] = a[tokens, k] . W     n = in_features,  k = out_features (:522-525)
 *   plan: built by pbs_blocksparse_matmul_plan from the (ptr, indices) pair the reference passes
 *         here, for the same transpose
 *
 * Differences from the reference entry point, all on purpose: `data` is always the packed data as
 * stored (no per-call transposed copy of the weights, :541-544); `out` is row-major [tokens, n]
 * and need not be zeroed (the reference wants a zeroed [n, tokens] buffer, :516); `bias` is NULL
 * or [n] and is added in the epilogue (the reference adds it in a separate pass,
 * block_sparse_linear.py:231-232); any tokens >= 0 is handled; work is launched on `stream`,
 * not on stream 0.
 */
int pbs_blocksparse_matmul(const void* dense_a, const void* data, const void* plan,
                           const void* bias, void* dense_out,
                           int64_t tokens, int n, int k, int nnz,
                           int transpose, int dtype, void* stream);

/*
 * The same product with an optional workspace.  The reference's reverse_matmul_ hands its kernel a
 * transposed copy of the packed data for one of the two directions, made on every call
 * (block_sparse.py:541-544: data.reshape(-1, 32, 32).transpose(1, 2).reshape(-1, 32).contiguous()).
 * The fastest bf16 kernel for patterns with many blocks per column wants the same for the forward
 * direction (every block with the contraction index along its rows); the library makes that copy in
 * `workspace`, on `stream`, before the product, when the caller provides one of
 * pbs_blocksparse_matmul_workspace_bytes() bytes (16-byte aligned device memory, contents
 * unspecified afterwards).  With workspace = NULL, or one that is too small, the call is
 * pbs_blocksparse_matmul: same results to the last bit of bf16 rounding of the same fp32 sums in a
 * different order, from a kernel that reads the data as stored.  ..._workspace_bytes() returns 0 when
 * no workspace would be used (fp32, the input-gradient direction, small or very sparse problems).
 */
size_t pbs_blocksparse_matmul_workspace_bytes(int64_t tokens, int n, int k, int nnz, int transpose, int dtype);
int pbs_blocksparse_matmul_ws(const void* dense_a, const void* data, const void* plan,
                              const void* bias, void* dense_out,
                              int64_t tokens, int n, int k, int nnz,
                              int transpose, int dtype,
                              void* workspace, size_t workspace_bytes, void* stream);

/*
 * dense^T x dense -> block-sparse (only the nonzero blocks are computed), packed like
 * `data`:  out[32b + j][i] = sum_t dense_a[t][32r + i] * dense_b[t][32c + j].
 * Replaces blocksparse_matmul_back_cutlass (native/block_sparse_native.cpp:18-29,
 * launcher native/block_sparse_cutlass_kernel_back.cu:118-160) as called by
 * matmul_with_output_sparse_support_ (block_sparse.py:606-655); result layout as in
 * cutlass/gemm/block_task_back.h:537-538.
 *
 *   dense_a [tokens, out_features] (grad_output), dense_b [tokens, in_features] (input),
 *   both row-major contiguous.  The pattern is given by the CSR pair
 *   (row_start_ends_a, cols_a) instead of the reference's `blocks` list so that a
 *   workgroup can find the blocks of its tile of W without scanning all of them.
 *   A caller of the reference's entry point has the pair at hand: the object that owns
 *   `blocks` registers row_start_ends_a and cols_a as buffers next to it
 *   (block_sparse.py:58-65), built from the same mask by build_indices (:125-153); a
 *   caller that holds nothing but a mask obtains all of them from pbs_build_indices.
 *   Every token is accumulated (the reference drops tokens % 32 when tokens > 32).
 *   `out` need not be zeroed.
 *
 * When the tile grid alone cannot fill the GPU the token range is split over
 * workgroups and the fp32 partial blocks are summed in a fixed order by a second
 * kernel; that needs `workspace` of pbs_blocksparse_matmul_back_workspace_bytes()
 * bytes (16-byte aligned device memory; may be NULL when that returns 0).
 */
size_t pbs_blocksparse_matmul_back_workspace_bytes(int64_t tokens, int out_features, int in_features,
                                                   int nnz, int dtype);
int pbs_blocksparse_matmul_back(const void* dense_a, const void* dense_b,
                                const int32_t* row_start_ends_a, const int32_t* cols_a,
                                void* data_out,
                                int64_t tokens, int out_features, int in_features, int nnz,
                                int dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same product with the arguments of the reference's entry point blocksparse_matmul_back_cutlass
 * (native/block_sparse_native.cpp:18-29; launcher native/block_sparse_cutlass_kernel_back.cu:118-160, which
 * picks one of four kernels by the two memory-order flags, :145-157), for a caller that holds what the
 * reference's call site holds (block_sparse.py:606-652): the two dense operands with a flag each, and the
 * `blocks` list.
 *
 *   a_row_major / b_row_major   1: the operand is [tokens, features] row-major (a "contiguous" torch tensor, the
 *                               reference's pytorch_contiguous_* = true); 0: it is [features, tokens] row-major,
 *                               i.e. its transpose is contiguous (block_sparse.py:480-494)
 *   blocks [nnz][2]             (block column, block row) of data block b, in any order (block_sparse.py:138-141)
 *
 * The CSR pair is derived from `blocks` on the device (three small kernels), and an operand given in the second
 * order is transposed on the device, both into `workspace`; then pbs_blocksparse_matmul_back runs.  All of it
 * is launched on `stream`.  workspace: 16-byte aligned device memory of
 * pbs_blocksparse_matmul_back_blocks_workspace_bytes() bytes (index arrays + transposed operands + the partial
 * sums of a split token range).  A caller that already holds row_start_ends_a / cols_a and row-major operands
 * saves those steps by calling pbs_blocksparse_matmul_back.
 */
size_t pbs_blocksparse_matmul_back_blocks_workspace_bytes(int64_t tokens, int out_features, int in_features, int nnz,
                                                          int dtype, int a_row_major, int b_row_major);
int pbs_blocksparse_matmul_back_blocks(const void* dense_a, int a_row_major, const void* dense_b, int b_row_major,
                                       void* data_out,
                                       int64_t tokens, int out_features, int in_features,
                                       const int32_t* blocks, int nnz,
                                       int dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * pbs_blocksparse_matmul_back for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same kernels and bit-identical results as pbs_blocksparse_matmul_back,
 * without the workspace pair: the fp32 partial sums of a split token range go to a device array of
 * PBS_NOALLOC_SCRATCH_BYTES (64 MiB) that is part of the library (every GPU the library is used on
 * holds its own copy until the process ends).  The call makes no hipMalloc/hipFree and calls no
 * allocating routine.
 *
 *   - A problem whose pbs_blocksparse_matmul_back_workspace_bytes() exceeds the array is rejected
 *     with PBS_ERR_SCRATCH before anything is launched (4096 x 4096 at density 0.25 with 16384
 *     tokens in bf16 needs exactly 64 MiB and fits).
 *   - Nothing in the array has to be cleared between calls: every word the reduction kernel reads
 *     is written by the product kernel of the same call first.
 *   - All calls on one GPU share that GPU's array, whatever their stream: two calls that overlap on
 *     one GPU race.  Order them on one stream, or use the workspace entry point for concurrent work.
 *   - The first call on a GPU looks up that GPU's address of the array (hipGetSymbolAddress).  A caller that is
 *     going to capture the call into a HIP graph calls pbs_blocksparse_matmul_back_noalloc_init() once per GPU,
 *     with that GPU current, before the capture begins; it does the lookup and nothing else.
 */
#define PBS_NOALLOC_SCRATCH_BYTES (64u << 20)
size_t pbs_blocksparse_matmul_back_noalloc_max_bytes(void);
int pbs_blocksparse_matmul_back_noalloc_init(void);
int pbs_blocksparse_matmul_back_noalloc(const void* dense_a, const void* dense_b,
                                        const int32_t* row_start_ends_a, const int32_t* cols_a,
                                        void* data_out,
                                        int64_t tokens, int out_features, int in_features, int nnz,
                                        int dtype, void* stream);

/*
 * Diagnostics.  Neither has a counterpart in the reference.
 *
 * pbs_protocol_failures: the bf16 kernels for large problems (dds16_kernel, ddsc_kernel) synchronise their waves
 * through progress words in LDS with bounded waits instead of barriers.  A wait that runs into its bound means a
 * broken protocol; the kernel then writes NaN into the results it could not vouch for and counts the event in a
 * device word.  This call copies the current GPU's count (since the library was loaded) to *count; it synchronises
 * the device.  The Python layer checks it after every product when PBS_DEBUG is set and raises.
 *
 * pbs_blocksparse_matmul_kernel_name / ..._back_kernel_name: which kernel(s) a call with these sizes runs
 * ("dds_kernel", "dds16_kernel", "ddsc_kernel"; "sdd_seg_kernel", "sdd_kernel", "sdd_bf16_kernel", with
 * " + sdd_reduce_kernel" when the token range is split), for benchmark labels.  "" for arguments the product
 * entry points reject.
 */
int pbs_protocol_failures(unsigned* count);
const char* pbs_blocksparse_matmul_kernel_name(int64_t tokens, int n, int k, int nnz, int transpose, int dtype,
                                               int with_workspace);
const char* pbs_blocksparse_matmul_back_kernel_name(int64_t tokens, int out_features, int in_features, int nnz,
                                                    int dtype);

#ifdef __cplusplus
}
#endif
#endif /* PBS_HIP_H */
