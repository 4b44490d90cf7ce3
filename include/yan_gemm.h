/* C ABI of the MI355X (gfx950) GEMM hot path: bf16 / fp16 dense GEMM and FP8 e4m3 block-scaled GEMM.
 *
 * Two ways in, both plain C with raw device pointers and sizes:
 *
 * 1. The ahead-of-time library libyan_gemm.so (yan_amd/csrc), declared below: every tile variant precompiled,
 *    sizes taken at run time. This is what a host that is not Python (or does not want a compiler at run time)
 *    binds.
 * 2. A JIT-built kernel.so, which exports exactly one symbol,
 *        void launch(<one parameter per argument>, int* __return_code);
 *    with tensors and streams passed as void* and bool/int/float by value. This is the boundary of the reference
 *    (yan/jit/template.py:121-149 generates it, yan/jit/runtime.py:54-68 calls it through ctypes). The two
 *    instantiations this path uses are spelled out as function-pointer types at the end of this header.
 *
 * Conventions shared by every entry point:
 *   - all matrices are row-major with the K dimension contiguous ("TN"/"NT": both operands K-major);
 *   - pointers are device pointers owned by the caller; nothing is allocated, freed or retained (the split-K entry points
 *     work in a caller-owned workspace, or, for the one that says so, in a device array the library holds);
 *   - work is enqueued on `stream` (a hipStream_t, NULL for the default stream) and NOT synchronised;
 *   - the return value is a hipError_t as int: 0 on success, hipErrorInvalidValue (1) for sizes the kernels do
 *     not take (they never fault on a bad size), or whatever the launch reported;
 *   - m == 0 or n == 0 is a successful no-op.
 */
#ifndef YAN_GEMM_H
#define YAN_GEMM_H

#if defined(__GNUC__)
#define YAN_API __attribute__((visibility("default")))
#else
#define YAN_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* c[m,n] = a[m,k] . b[n,k]^T, bf16 in, fp32 accumulate, bf16 out (round to nearest even).
 * Requires n % 4 == 0, k % 8 == 0, (m rounded up to the tile's rows, at most 256) * k * 2 < 2^31 bytes, same for n,
 * and 256 * n * 2 < 2^31 bytes (output stores address one tile with 32-bit offsets).
 * Replaces gemm_fp16_tn -> gemm_tn<128,128,3> of the reference (yan/jit_kernels/cute_gemm.py:21-64,
 * yan/include/gemm/cute_gemm.cuh:262-378), with the bf16 dtype and fp32 accumulation. */
YAN_API int yan_gemm_bf16_tn(int m, int n, int k, const void* a, const void* b, void* c, void* stream);

/* Same contraction for IEEE fp16 in / fp16 out, fp32 accumulate (the reference's dtype, cute_gemm.py:26). */
YAN_API int yan_gemm_fp16_tn(int m, int n, int k, const void* a, const void* b, void* c, void* stream);

/* The two dense GEMMs with K split over 2 to 4 workgroups per output tile where that pays: problems whose tiles would leave
 * compute units idle and whose K is long (the smallest dense tile holds 64 weight rows, so 64 x 4096 x 7168 runs on 64
 * workgroups; in four parts it runs on 256 and takes 16 us instead of 37). The parts leave fp32 partial sums in `workspace`;
 * the part that arrives last adds them up in the order of their K ranges (results are repeatable to the bit) and stores the
 * tile. Within the tolerance of the plain entry points, not bit-identical to them; every other problem runs exactly as
 * through the plain entry points. `workspace` / `workspace_bytes`: as for yan_gemm_fp8_fp8_bf16_nt_split_k below (one
 * workspace serves all three). The reference's dense launcher has no split (yan/include/gemm/cute_gemm.cuh:262-378). */
YAN_API int yan_gemm_bf16_tn_split_k(int m, int n, int k, const void* a, const void* b, void* c, void* stream, void* workspace,
                             long long workspace_bytes);
YAN_API int yan_gemm_fp16_tn_split_k(int m, int n, int k, const void* a, const void* b, void* c, void* stream, void* workspace,
                             long long workspace_bytes);

/* c = alpha * a . b^T + beta * c in fp32 (fp32 MFMA accumulation).
 *   a  m x k with M contiguous: element (i, kk) at a[i + kk*lda];   b  n x k with N contiguous: b[j + kk*ldb];
 *   c  m x n row-major: c[i*ldc + j].  beta == 0 does not read c.
 * Requires m, n, lda, ldb, ldc multiples of 4, lda >= m, ldb >= n, ldc >= n, 16-byte aligned pointers and
 * ((k + 1024) * lda + 256) * 4 < 2^31 bytes, same for ldb (the kernel prefetches up to 8 k-tiles of 128 k-rows past
 * the end through a descriptor with 32-bit offsets; those rows read as zero). k == 0 scales c by beta.
 * Replaces gemm_float_nt -> gemm_nt of the reference (yan/jit_kernels/simple_gemm.py:18-57,
 * yan/include/gemm/simple_gemm.cuh:194-247), same argument order and memory convention. */
YAN_API int yan_gemm_float_nt(int m, int n, int k, float alpha, const float* a, int lda, const float* b, int ldb,
                              float beta, float* c, int ldc, void* stream);

/* out[i,j] = bf16( sum_kb lhs_scales(i,kb) * rhs_scales[j/128][kb] * sum_{t<128} lhs[i][128kb+t] * rhs[j][128kb+t] )
 *   lhs        e4m3 (OCP, max 448) [m,k] row-major
 *   lhs_scales fp32, element (i,kb) at lhs_scales[i*lhs_scales_stride_m + kb*lhs_scales_stride_k]
 *              (row-major: strides (k/128, 1); token-contiguous as DeepGEMM callers pass it: (1, m))
 *              Both give the same bits. Large problems (256-row tiles) run 13-18 % faster on token-contiguous scales:
 *              a wave reads one scale per lane and k-tile, in the row-major layout a cache line each.
 *   rhs        e4m3 [n,k] row-major;  rhs_scales fp32 [ceil(n/128)][k/128] row-major
 *   out        bf16 [m,n] row-major
 * Requires k % 128 == 0, n % 4 == 0; m arbitrary; (m rounded up to the tile's rows, at most 256) * k < 2^31 bytes, same
 * for n; 256 * n * 2 < 2^31 bytes; the last activation scale at an offset below 2^28 elements.
 * `num_sms` is the caller's compute-unit cap, the grid size of the reference's persistent kernel
 * (yan/include/gemm/fp8_gemm.cuh:40, yan/jit_kernels/gemm.py:26-30): 0, or a value of at least the device's compute
 * units, starts one workgroup per output tile; a smaller value starts that many workgroups (rounded down to a
 * multiple of 8 from 8 up), each walking several tiles, and is also the number of compute units the tile choice
 * plans for. Results do not depend on it. The grouped entry points below take it in the same sense.
 * Nothing is allocated and no state is kept between calls.
 * Replaces the FP8 entry the reference only sketches: template yan/jit_kernels/gemm.py:9-31, kernel
 * yan/include/gemm/fp8_gemm.cuh:40-196. */
YAN_API int yan_gemm_fp8_fp8_bf16_nt(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                             long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales, void* out,
                             int m, int n, int k, void* stream, int num_sms);

/* The same GEMM with K split over 2 to 4 workgroups per output tile where that pays: problems whose tiles would leave
 * compute units idle and whose K is long (m up to a few hundred, k from about 4096: 64 x 4096 x 7168 runs 64 x 64 tiles in
 * four parts). The parts leave fp32 partial sums in `workspace`; the part that arrives last adds them up in the order of
 * their K ranges, so a result does not depend on which part that was, and stores the tile. Results are within the
 * tolerance of the plain entry point but not bit-identical to it (a different order of summation); every other problem
 * runs exactly as through the plain entry point.
 *   workspace        device memory of at least yan_gemm_split_k_workspace_bytes() bytes (16.0 MB), whose first
 *                    yan_gemm_split_k_counter_bytes() bytes (arrival counters) the caller zero-fills once, before the
 *                    first call; every call leaves them zero again, so one workspace serves calls of any shapes;
 *   workspace_bytes  its size; less than the problem's plan needs is hipErrorInvalidValue.
 * Calls that share a workspace must not overlap on the device (same stream, or otherwise ordered).
 * This is the `split` half of the reference's tile/split heuristics, which its template leaves to the caller's keys
 * (yan/jit_kernels/gemm.py:13-18); yan_gemm_select_split_k below says what a problem gets. */
YAN_API long long yan_gemm_split_k_workspace_bytes(void);
YAN_API long long yan_gemm_split_k_counter_bytes(void);
YAN_API int yan_gemm_fp8_fp8_bf16_nt_split_k(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                                     long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales, void* out,
                                     int m, int n, int k, void* stream, int num_sms, void* workspace,
                                     long long workspace_bytes);

/* The split-K GEMM above for callers that cannot allocate or own a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the workspace is a device array inside the library, 16.0 MB
 * (yan_gemm_split_k_workspace_bytes()) on every GPU the library runs on, held until the process ends; the call
 * allocates nothing and frees nothing. Same arguments, same plans and same bits as yan_gemm_fp8_fp8_bf16_nt_split_k. A problem
 * whose plan needed more than the array holds would return hipErrorInvalidValue without launching (no plan for up to 256
 * compute units does). Every call on a GPU uses that GPU's one array, on whatever stream or host thread: calls that
 * overlap on the device race; calls on one stream, or otherwise ordered, are safe, and each leaves the counters at zero.
 * It has no counterpart in the reference. */
YAN_API int yan_gemm_fp8_fp8_bf16_nt_static(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                                    long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales, void* out,
                                    int m, int n, int k, void* stream, int num_sms);

/* Puts the arrival counters of a split-K workspace back to zero, on `stream` (a small fill kernel, so the call may be
 * captured into a graph). `workspace` NULL names the library's own array, the one yan_gemm_fp8_fp8_bf16_nt_static uses on
 * the current GPU. The counters are zero after every split-K launch that ran to its end, so an ordinary caller needs this
 * once at most (instead of zero-filling a fresh workspace itself). Call it before reusing a workspace after anything that
 * may have left a launch half done: a split-K call that returned non-zero, calls that overlapped on one workspace, a
 * device reset. Partial sums need no clearing. It has no counterpart in the reference (its kernels keep no state). */
YAN_API int yan_gemm_split_k_reset(void* workspace, void* stream);

/* Grouped (mixture-of-experts) forms of the FP8 GEMM: group g has its own weights rhs[g] ([n,k] e4m3) and scale table
 * rhs_scales[g] ([ceil(n/128)][k/128]); both arrays are contiguous over g. Arithmetic per row as above.
 * They fill in the reference's GemmType::GroupedContiguous / GroupedMasked and `int* grouped_layout` hooks
 * (yan/include/gemm/scheduler.cuh:7-11,31-48, yan/include/gemm/fp8_gemm.cuh:41), for which it has no entry point.
 *
 * contiguous: lhs [m,k] holds the rows of all groups one after the other, every group padded to a multiple of 128 rows
 *   (get_m_alignment_for_contiguous_layout, yan/jit_kernels/utils.py:46-55), so m % 128 == 0; m_indices[i] (device,
 *   int32 [m]) is the group of row i, constant over each aligned block of 128 rows; a negative value marks a block of
 *   padding rows, whose rows of `out` are not written. Groups of a few hundred rows that are padded to multiples of 256 rows
 *   run up to 17 % faster than others (no 256-row tile then holds two groups; see yan_gemm_select_tile op 4). */
YAN_API int yan_m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                                                  long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales,
                                                  void* out, const int* m_indices, int num_groups, int m, int n, int k,
                                                  void* stream, int num_sms);

/* masked: lhs [num_groups][m_max][k], out [num_groups][m_max][n], both contiguous; scale (g,i,kb) of lhs at
 *   lhs_scales[g*stride_g + i*stride_m + kb*stride_k]; masked_m (device, int32 [num_groups]) says how many leading rows
 *   of each group are valid; the other rows of `out` are not written. expected_m > 0 is a hint for the tile choice
 *   and the launch order (the tile rows below it come first); results do not depend on it. */
YAN_API int yan_m_grouped_gemm_fp8_fp8_bf16_nt_masked(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_g,
                                              long long lhs_scales_stride_m, long long lhs_scales_stride_k, const void* rhs,
                                              const float* rhs_scales, void* out, const int* masked_m, int num_groups,
                                              int m_max, int expected_m, int n, int k, void* stream, int num_sms);

/* Quantisers producing the GEMM's operands in one pass over HBM: amax over the group clamped at 1e-4,
 * q = e4m3(x * (448 / amax)) with round to nearest even, scale = amax / 448, both quotients correctly rounded fp32
 * divisions (the op chain callers of this convention type in torch, which itself rounds 448 / amax an ulp differently
 * for some amax). Sources are bf16 (x_is_fp32 == 0) or fp32, row-major, k % 128 == 0.
 * per-token: groups of 1 x 128; scale (i, kb) is written to scales[i*scales_stride_m + kb*scales_stride_k]
 *            ((k/128, 1) for row-major, (1, m) for the token-contiguous layout the GEMM reads fastest).
 * per-block: groups of 128 x 128 (a ragged last block of rows uses the rows that exist); scales [ceil(n/128)][k/128].
 * They produce what the reference's operand names lhs/lhs_scales and rhs/rhs_scales stand for
 * (yan/jit_kernels/gemm.py:23-30); the reference has no quantiser of its own. */
YAN_API int yan_per_token_cast_to_fp8(const void* x, int x_is_fp32, void* q, float* scales, long long scales_stride_m,
                              long long scales_stride_k, int m, int k, void* stream);
YAN_API int yan_per_block_cast_to_fp8(const void* w, int w_is_fp32, void* q, float* scales, int n, int k, void* stream);

/* Macro tile the library uses for a problem: op 0 = dense 16-bit, 1 = FP8 block-scaled, 2 = FP8 grouped contiguous
 * (m = total rows, and `k` carries the number of groups instead of the depth), 3 = fp32. Writes BLOCK_M / BLOCK_N.
 * op 4 (m, `k` as for op 2): 256 x 256 when the contiguous entry point runs the kernel that holds 256 x 256 and 128 x 256
 * tiles and decides on the device, from m_indices, which tile rows run as which (groups of 256 to 2047 rows on average),
 * 0 x 0 when it runs the tile op 2 names.
 * For ops 0 and 1 with few activation rows the answer is (16 * atoms, 16): the weight-streaming kernels.
 * Host-only (no device call). Stands where the reference leaves tile choice to the caller's keys
 * (yan/jit_kernels/cute_gemm.py:41, yan/jit_kernels/gemm.py:13-16). Returns 0, or 1 for an unknown op. */
YAN_API int yan_gemm_select_tile(int op, int m, int n, int k, int num_cus, int* block_m, int* block_n);

/* Split-K plan of the dense 16-bit GEMM (op 0) or the plain FP8 GEMM (op 1) on `num_cus` compute units: writes the tile
 * and the number of parts, or block_m = block_n = 0 and split_k = 1 when K is not split (then yan_gemm_select_tile names
 * the tile). Host-only. Returns 0, or 1 for another op, a null pointer or num_cus <= 0. */
YAN_API int yan_gemm_select_split_k(int op, int m, int n, int k, int num_cus, int* block_m, int* block_n, int* split_k);

/* "yan-gemm gfx950 <n> dense + <n> fp32 + <n> fp8 tile variants + <n> weight-streaming fp8 variant + ...". */
YAN_API const char* yan_gemm_version(void);

/* The JIT boundary, for reference: signatures of `launch` in the kernel.so of each op
 * (argument lists of yan/jit_kernels/cute_gemm.py:55-59 and yan/jit_kernels/gemm.py:23-30). The FP8 form with the
 * reference's nine arguments takes token-contiguous activation scales (element (i, kb) at kb * m + i); the strided form
 * is this build's addition for every other layout, with the two strides in elements. */
typedef void (*yan_jit_launch_dense_fn)(int m, int n, int k, void* A, void* B, void* C, void* stream, int* return_code);
typedef void (*yan_jit_launch_fp8_fn)(void* lhs, void* lhs_scales, void* rhs, void* rhs_scales, void* out, int m,
                                      void* stream, int num_sms, int smem_size, int* return_code);
typedef void (*yan_jit_launch_fp8_strided_fn)(void* lhs, void* lhs_scales, void* rhs, void* rhs_scales, void* out, int m,
                                              void* stream, int num_sms, int smem_size, int lhs_scales_stride_m,
                                              int lhs_scales_stride_k, int* return_code);

#ifdef __cplusplus
}
#endif
#endif /* YAN_GEMM_H */
