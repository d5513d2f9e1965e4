/* C ABI of libhx_kernels.so — hand-written gfx950 (MI355X) kernels behind the three Helion example
 * entry points fp8_gemm, fp8_attention_kernel and moe_matmul_ogs, and of their 16-bit siblings matmul,
 * matmul_split_k and attention.
 *
 * Conventions (all functions):
 *   - plain pointers and sizes only; every pointer is DEVICE memory owned by the caller;
 *   - the library never allocates, frees or retains device memory; scratch comes in through the
 *     `workspace` arguments (sizes from the hx_*_workspace_bytes queries);
 *   - kernels are enqueued on `stream` (a hipStream_t passed as void*; NULL = default stream),
 *     nothing synchronises the host;
 *   - return 0 on success; a negative value is an argument/shape error detected before any
 *     launch; a positive value is the hipError_t of a failed launch.  hx_last_error() returns a
 *     thread-local message for the last non-zero return.
 */
#ifndef HX_KERNELS_H
#define HX_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type tags used by out_dtype / dtype arguments */
enum {
  HX_F16 = 0,
  HX_BF16 = 1,
  HX_F32 = 2,
  HX_E4M3 = 3 /* OCP float8_e4m3fn */
};

/* error codes (negative returns) */
enum {
  HX_ERR_BAD_ARG = -1,     /* null pointer, negative size, unknown dtype tag */
  HX_ERR_UNSUPPORTED = -2, /* shape/stride/alignment outside what the kernels handle */
  HX_ERR_WORKSPACE = -3    /* workspace missing or too small */
};

int hx_version(void);
const char* hx_last_error(void);

/* Opt-in kernel paths.  A path listed here has passed the CPU-side checks (the kernel source executed lane by lane
 * on the host against the oracle, with every operand access bounds-checked) but has not yet been run on an MI355X, so
 * it is compiled in and off by default: calls take the kernels that have.  hx_set_features replaces the process-wide
 * mask (returns the previous one); its initial value is the environment variable HX_FEATURES (a number).  The
 * hx_*_path and hx_*_workspace_bytes queries answer for the mask in force when they are called. */
enum {
  HX_FEATURE_SKINNY_ROWMAJOR = 1, /* hx_fp8_gemm, M <= 32, row-major b (ldb_n == 1), K % 1024 == 0, N % 16 == 0: b is
                                    streamed in place (path 6) instead of being transposed through the workspace */
  HX_FEATURE_FP8_GEMM_ANY_K = 2, /* hx_fp8_gemm with K % 16 != 0 (or rows / pointers that are not 16-byte aligned) and a
                                    workspace: the operands are copied once into it as K-contiguous rows zero-padded to
                                    the next multiple of 16 and the MFMA kernels run on the copies, where the plain fp32
                                    kernel ran before (hx_fp8_gemm_path still answers 0 for such a call) */
  HX_FEATURE_ATTENTION_D256 = 4, /* hx_fp8_attention with head dim 256 on the MFMA kernel (hx_fp8_attention_path 1)
                                    instead of the one-workgroup-per-query-row kernel */
  HX_FEATURE_FP8_GEMM_PERSISTENT = 8, /* hx_fp8_gemm on the 256x256 tile kernel with at least two tiles per CU, K % 256 == 0
                                    and a 16-bit output: persistent workgroups whose epilogue runs inside the next tile's
                                    first k-tile (path 7) */
  HX_FEATURE_FP8_GEMM_DECODE_RING = 16, /* hx_fp8_gemm with 33..256 rows and a column-major b: the weight-streaming kernel with
                                    separate LDS rings and wave streams for a and b (path 8 where path 5 ran before) */
  HX_FEATURE_ROUTING_WIDE = 32, /* hx_moe_routing with 513..2048 experts (HX_ERR_UNSUPPORTED before): the same kernels with
                                    LDS tables for 2048 experts */
  HX_FEATURE_MATMUL_PERSISTENT = 128, /* hx_matmul on the 256x256 tile kernel with a row-major b, no epilogue, a 16-bit output,
                                    M % 256 == 0, N % 256 == 0, K % 128 == 0, K >= 256 and at least two tiles per CU: persistent
                                    workgroups, as HX_FEATURE_MOE_PERSISTENT (hx_matmul_path 2) */
  HX_FEATURE_MOE_PERSISTENT = 64, /* the grouped GEMM's 256-row tiles (hx_moe_path 3) with N % 256 == 0, K % 128 == 0, K >= 256
                                    in persistent workgroups whose epilogue runs inside the next tile's first k-tile
                                    (hx_moe_path 6); hx_moe_workspace_bytes grows by about 1 KB while it is on */
  HX_FEATURE_MOE_ANY_SHAPE = 256 /* hx_moe_grouped_gemm with an odd K or N % 8 != 0 and a workspace of
                                    hx_moe_workspace_bytes_shape(T, K, N, E) bytes: the operands are copied once into it,
                                    zero-padded to multiples of 8, and the MFMA kernels run on the copies where the fp32
                                    kernel ran before (hx_moe_path still answers 0 for such a call) */
};
unsigned hx_set_features(unsigned mask);
unsigned hx_get_features(void);

/* Replaces the device side of `fp8_gemm(x, y)` (reference: examples/fp8_gemm.py:29-57, whose
 * generated launcher is test/test_examples.expected:821-841) and of its baseline
 * `torch._scaled_mm` call (examples/fp8_gemm.py:61-78).
 *   c[m,n] = cast( (sum_k f32(a[m,k]) * f32(b[k,n])) * (scale_a*scale_b) )
 * a: [M,K] e4m3fn, element (m,k) at a[m*lda + k].
 * b: [K,N] e4m3fn, element (k,n) at b[k*ldb_k + n*ldb_n]  (ldb_k==1: "column-major" B, the layout
 *    torch._scaled_mm wants; ldb_n==1: row-major B as the example's check() feeds).
 * c: [M,N] of out_dtype (HX_F16 = reference default, HX_BF16, HX_F32), element (m,n) at c[m*ldc+n].
 * scale_a/scale_b: device pointers to one fp32 each, or NULL for 1.0 (the reference hard-codes
 *    1.0, helion/language/matmul_ops.py:232-233).
 * hx_fp8_gemm_path: 0 plain kernel (or a row-major b transposed through the workspace), 1 256x256 tiles, 2 decode kernel,
 * 3 256x256 tiles with guarded edges / K tail, 4 256x256 tiles on a row-major b, 5 128-column tiles, 6 decode kernel on a
 * row-major b (opt-in), 7 256x256 tiles in persistent workgroups (opt-in), 8 decode batch of 33..256 rows with separate
 * a / b rings (opt-in).
 * Chooses between the 256x256 MFMA tile kernel (with guarded edge tiles when M or N is ragged or K is not a multiple
 * of 128 — K % 16 == 0 suffices, the last k-tile is zero-padded in LDS; it reads a column-major B directly and a
 * row-major B through transposing LDS loads), the skinny (M<=16, or M<=32 with K<=8192) wave-split-K kernel
 * and a bounds-checked general kernel from the shape, strides and alignment.
 * workspace: optional device scratch of hx_fp8_gemm_workspace_bytes(...) bytes, 16-byte aligned, any content; it
 *    belongs to the call until its kernels have finished (two launches in flight at once need two workspaces).
 *    A decode call (path 2) with at least 12 column groups of 16 per CU hands its last groups out by ticket through the
 *    first 8 bytes (any content before, zero after).  Sharing that word between two launches in flight is the misuse
 *    above: a workgroup then waits a few milliseconds at most for its launch's tag, stops drawing, and stores a value with
 *    bit 63 set into bytes 8..15.  The library only ever sets those bytes; a caller who wants the record zeroes them
 *    before the call and reads them after it.
 *    With HX_FEATURE_SKINNY_ROWMAJOR on, a row-major b for M <= 32 with K % 1024 == 0 and N % 16 == 0 is streamed in
 *    place (path 6) and needs scratch only for fp32 partial sums when few column groups meet a long K. */
int hx_fp8_gemm(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda,
                int64_t ldb_k, int64_t ldb_n, int64_t ldc, const float* scale_a, const float* scale_b,
                int out_dtype, void* workspace, size_t workspace_bytes, void* stream);
/* Scratch hx_fp8_gemm can use for these arguments.  Row-major B that the tile kernel cannot read in place (M <= 16,
 * or N / the row stride not a multiple of 16): N*K bytes for a one-off transpose into the K-contiguous layout,
 * without which such a B runs on the slow general kernel.  Column-major B: splits*M*N*4 bytes when the 128-column
 * tile kernel would cut K into `splits` pieces (its tiles occupy less than half of the CUs and K is at least 16
 * k-tiles long; at most 32 MB), without which it runs unsplit; 16 bytes for a decode call (M <= 16, K <= 8192) with at
 * least 12 column groups of 16 per CU: the word through which the last groups are handed out to whichever workgroup is
 * free (needs no initialisation, is left zero), without which every workgroup takes a fixed share.  0 otherwise. */
size_t hx_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t ldb_k, int64_t ldb_n);

/* Which kernel hx_fp8_gemm would launch for these arguments: 0 general (or, given a workspace, transpose + fast
 * path), 1 tile256, 2 skinny, 3 tile256 with guarded edge tiles (M or N not a multiple of 256), 4 tile256 reading a
 * row-major B in place (edges included), 5 the 128-column tile kernel (column-major B, K % 128 == 0, taken while its
 * rounds of tiles are estimated to finish before those of 256x256 tiles: decode batches of 33..256 rows, small and
 * mid-size products).
 * (Diagnostic; lets tests assert that the fast paths are the ones exercised.) */
int hx_fp8_gemm_path(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n,
                     int64_t ldc, const void* a, const void* b, const void* c);

/* Replaces the device side of `fp8_attention_kernel(q, k, v, batch, heads)` (reference:
 * examples/fp8_attention.py:22-106; generated kernel test/test_examples.expected:718-766).
 * q,k: [BH,S,D] e4m3fn contiguous; v: logically [BH,D,S] e4m3fn, element (bh,d,s) at
 *   v[bh*S*D + d*v_stride_d + s*v_stride_s], in one of two physical layouts per head:
 *   (v_stride_d, v_stride_s) = (S, 1): [D][S] contiguous ("pre-transposed");
 *   (v_stride_d, v_stride_s) = (1, D): [S][D], which is what the reference's own preprocessing produces
 *   (examples/fp8_attention.py:119-121: `v.permute(0,1,3,2).to(e4m3)` keeps the memory order of [B,H,S,D]);
 *   neither needs a copy: the second is read with transposing LDS loads.
 * out: [BH,S,D] contiguous (== [batch,heads,S,D]) of out_dtype HX_E4M3 (reference) or HX_F32.
 * exact_max != 0: two passes, P is quantised to e4m3 against the exact row max (bit-faithful to
 *   the reference's ref-eager execution); exact_max == 0: one pass, online softmax, P quantised
 *   against the running max (what the reference's compiled kernel does).
 * scale_dim: the head dimension the softmax scale 1/sqrt(.) is taken from; 0 = D.  (A caller whose head dimension is
 *   not 64 or 128 can zero-pad q, k and v to one of them, pass the true one here and drop the padded output columns:
 *   zero columns change neither q.k nor the other output columns.  The Python op does this.)
 * MFMA kernel: D == 128 or 64, any S (a partial last key tile is masked), 16-byte aligned pointers, v in one of the
 * two layouts above (the [D][S] layout needs S % 16 == 0: its rows are fetched in 16-byte pieces).  Every other shape
 * with D <= 256 and BH < 65536 (and any v strides within a head) runs a plain kernel that always computes the
 * exact-max form.  hx_fp8_attention_path: 1 = the MFMA kernel would run, 0 = the plain one. */
int hx_fp8_attention(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t S, int64_t D,
                     int64_t scale_dim, int64_t v_stride_d, int64_t v_stride_s, int out_dtype, int exact_max, void* stream);
int hx_fp8_attention_path(int64_t BH, int64_t S, int64_t D, int64_t v_stride_d, int64_t v_stride_s, const void* q,
                          const void* k, const void* v, const void* out);

/* Replaces the device side of `moe_matmul_ogs(A, W, expert_token_counts, expert_token_offsets,
 * sorted_to_orig_token_idx, max_T_per_expert_tensor)` (reference: examples/moe_matmul_ogs.py:25-80;
 * semantics = moe_matmul_ogs_reference, :125-148).
 *   for each expert e, for i in [0, counts[e]):  r = idx[offsets[e]+i];  C[r,:] = cast(A[r,:] @ W[e])
 *   rows of C that no expert covers are set to zero.
 * A: [T,K] row-major; W: [E,K,N] row-major (N contiguous); C: [T,N] row-major; dtype HX_BF16 or
 * HX_F16 for all three; counts [E], offsets [E+1], idx [T] are int32 device arrays.
 * max_T (the numel of the reference's dummy tensor) is accepted for signature parity and is only
 * validated (>= 0); the tile table is built on the device from counts/offsets.
 * workspace: hx_moe_workspace_bytes(T, E) bytes, 16-byte aligned.
 * MFMA kernels: K even and N % 8 == 0, 16-byte aligned pointers, A below 4 GB; a K that is not a multiple of 64 gets a
 * zero-filled last k-tile, and a K that is not a multiple of 8 (rows of A only 4-byte aligned, e.g. the K = 500 of the
 * reference's own check, examples/moe_matmul_ogs.py:186) has A fetched in 4-byte pieces.  Anything else (odd K,
 * N % 8 != 0) runs an fp32-FMA kernel.  hx_moe_path (a_div = 1 for this entry point): 0 = the FMA kernel, 1 / 2 / 3 =
 * MFMA kernel with 32- / 128- / 256-row tiles, 4 = 128-row tiles with a partial last k-tile, 5 = the same with A in
 * 4-byte pieces, 6 = the 256-row tiles in persistent workgroups (opt-in, HX_FEATURE_MOE_PERSISTENT). */
int hx_moe_grouped_gemm(const void* A, const void* W, void* C, const int32_t* counts,
                        const int32_t* offsets, const int32_t* idx, int64_t T, int64_t K, int64_t N,
                        int64_t E, int64_t max_T, int dtype, void* workspace, size_t workspace_bytes,
                        void* stream);
size_t hx_moe_workspace_bytes(int64_t T, int64_t E);
/* The same, plus room for the padded copies of HX_FEATURE_MOE_ANY_SHAPE when that feature is on and the shape needs them
 * (otherwise equal to hx_moe_workspace_bytes(T, E)).  No counterpart in the reference. */
size_t hx_moe_workspace_bytes_shape(int64_t T, int64_t K, int64_t N, int64_t E);
int hx_moe_path(int64_t T, int64_t K, int64_t N, int64_t E, int64_t a_div, const void* A, const void* W, const void* C);

/* hx_moe_grouped_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, checks, kernels and
 * results as hx_moe_grouped_gemm, minus the workspace: the tile table and the row-covered flags live in a 256 KiB
 * device array built into the library (one copy per GPU, held until the process ends), whose address is looked up
 * on the first call on each device.  Calls neither hipMalloc nor hipFree nor anything that allocates.
 * Limits: T <= HX_MOE_STATIC_MAX_ROWS and E <= HX_MOE_STATIC_MAX_EXPERTS, otherwise HX_ERR_UNSUPPORTED and nothing
 * is launched.  Every call on a GPU uses that GPU's one array (each call rewrites the part it reads, so nothing
 * carries over from the previous call): two calls that overlap in time on one GPU -- different streams, or
 * different host threads -- race on it; calls on one stream are ordered and safe. */
enum { HX_MOE_STATIC_MAX_ROWS = 131072, HX_MOE_STATIC_MAX_EXPERTS = 1024 };
int hx_moe_grouped_gemm_static(const void* A, const void* W, void* C, const int32_t* counts, const int32_t* offsets,
                               const int32_t* idx, int64_t T, int64_t K, int64_t N, int64_t E, int64_t max_T, int dtype,
                               void* stream);

/* Replaces the tensor ops of `moe_matmul_ogs_helion_kernel_args_gen(A, W, top1_expert_per_token)` (reference:
 * examples/moe_matmul_ogs.py:84-121) with one kernel and no host synchronisation:
 *   idx = argsort(expert_ids, stable=True); counts = bincount(expert_ids, minlength=E);
 *   offsets = [0, cumsum(counts)]; *max_count = max(counts)   (the reference's `.item()` value, left on the device).
 * expert_ids: [T] device array of int32 (ids_are_int64 == 0) or int64; counts [E], offsets [E+1], idx [T],
 * max_count [1] are int32 device arrays.  Ids outside [0, E) are skipped: their rows appear in no expert's list,
 * offsets[E] is then < T and idx[offsets[E]..T) is filled with -1.  Supported: E <= 512 (E <= 2048 with HX_FEATURE_ROUTING_WIDE), T < 2^31 - 8192.
 * workspace: hx_moe_routing_workspace_bytes(T, E) bytes of device scratch (0 up to 32768 rows, where one workgroup
 * does the whole job in one launch); with less, larger inputs also run on that one workgroup, correct but slow. */
int hx_moe_routing(const void* expert_ids, int ids_are_int64, int64_t T, int64_t E, int32_t* counts, int32_t* offsets,
                   int32_t* idx, int32_t* max_count, void* workspace, size_t workspace_bytes, void* stream);
size_t hx_moe_routing_workspace_bytes(int64_t T, int64_t E);

/* Top-k form of the same path, without the reference caller's `A.repeat_interleave(top_k, 0)` copy and without
 * its host synchronisation: routes on the device (hx_moe_routing) and runs the grouped GEMM with row r of C
 * computed from row r / top_k of A_tok.
 *   A_tok: [T_tok, K]; expert_ids: [T_tok*top_k] (row r = token r / top_k, slot r % top_k); W: [E,K,N];
 *   C: [T_tok*top_k, N]; rows whose id is outside [0, E) are zero.
 * With top_k == 1 this is moe_matmul_ogs(A, W, *args_gen(A, W, expert_ids)) (examples/moe_matmul_ogs.py:25-121).
 * workspace: hx_moe_topk_workspace_bytes(T_tok, top_k, E) bytes, 16-byte aligned. */
int hx_moe_topk_matmul(const void* A_tok, const void* W, void* C, const void* expert_ids, int ids_are_int64,
                       int64_t T_tok, int64_t top_k, int64_t K, int64_t N, int64_t E, int dtype, void* workspace,
                       size_t workspace_bytes, void* stream);
size_t hx_moe_topk_workspace_bytes(int64_t T_tok, int64_t top_k, int64_t E);

/* `x.to(torch.float8_e4m3fn)` on the device for fp16 / bf16 / fp32 sources, optionally times *multiplier (a device
 * fp32, NULL = 1): dst[i] = e4m3(src[i] * m), round to nearest even, |v| <= 464 gives at most 448, larger or NaN
 * gives NaN (what torch's cast does).  The cast of examples/fp8_attention.py:113-121.  src_dtype: HX_F16, HX_BF16,
 * HX_F32; src and dst 16-byte aligned; any n. */
int hx_cast_e4m3(const void* src, void* dst, int64_t n, int src_dtype, const float* multiplier, void* stream);

/* The three casts of `preprocess_fp8_attention_inputs(q, k, v)` (reference: examples/fp8_attention.py:110-133) in one
 * launch: q8, k8, v8 = e4m3(q), e4m3(k), e4m3(v), n elements each, element order unchanged.  The reference permutes v
 * to [B,H,D,S] before its cast, which changes strides but not memory order; the caller takes the same view of v8
 * (strides (S*D, 1, D)) and hx_fp8_attention reads it in place. */
int hx_fp8_attention_preprocess(const void* q, const void* k, const void* v, void* q8, void* k8, void* v8, int64_t n,
                                int src_dtype, void* stream);

/* Per-tensor quantisation for the scaled GEMM (the reference's baseline call passes unit scales,
 * examples/fp8_gemm.py:74-78; this produces real ones; no counterpart function in the reference):
 *   amax = max|src|;  *scale_out = amax / 448 (1 if amax == 0);  dst[i] = e4m3(src[i] * (448 / amax))
 * so that dst * scale_out ~ src and hx_fp8_gemm(..., scale_a = scale_out, ...) undoes the scaling.  A NaN in src
 * makes the scale NaN.  scale_out: one device fp32.  workspace: hx_fp8_quantize_workspace_bytes(n) bytes, 16-byte
 * aligned.  Three launches (partial maxima, final reduction, cast), no host synchronisation. */
int hx_fp8_quantize(const void* src, void* dst, int64_t n, int src_dtype, float* scale_out, void* workspace,
                    size_t workspace_bytes, void* stream);
size_t hx_fp8_quantize_workspace_bytes(int64_t n);

/* Dense matmul with a fused epilogue — the reference's `matmul(x, y, epilogue)` (examples/matmul.py:25-56) and
 * `matmul_split_k(x, y, epilogue)` (examples/matmul_split_k.py:30-68) for the epilogues its examples and tests use
 * (identity, `acc + bias[tile[1]]`, `relu(acc + bias[tile[1]])`: examples/matmul.py:96-119, test/test_examples.py:143-200):
 *   c[M,N] = cast( act( fp32(a[M,K]) @ fp32(b[K,N]) + bias[N] ) ),  fp32 accumulation, act = relu if `relu` else identity.
 * in_dtype: HX_BF16 / HX_F16 (MFMA tile kernel when b is row-major (ldb_n == 1) or column-major (ldb_k == 1, e.g. the
 * transpose of a linear layer's [N, K] weight), K % 64 == 0, N % 8 == 0, lda % 8 == 0, its leading dimension % 8 == 0,
 * ldc % 4 == 0 and all pointers are 16-byte aligned) or HX_F32 (plain fp32 kernel, as is everything the
 * tile kernel does not cover).  out_dtype: in_dtype, or HX_F32 for the raw accumulator an arbitrary epilogue can be
 * applied to by the caller.  bias: null or [N] in in_dtype or HX_F32 (bias_dtype).
 * split_k: 1 = every workgroup runs the whole K; n > 1 = K split n ways (fewer if K / 64 < n); 0 = the library picks
 * (splits only while the output tiles alone do not fill the chip).  Splits go through fp32 partial sums in the
 * workspace (hx_matmul_workspace_bytes(...) bytes, 16-byte aligned; 0 for one split) and are summed in a fixed order,
 * with the epilogue applied to the whole sum: every split count gives the reference's one-split (eager) result up to
 * fp32 summation order.  hx_matmul_splits tells the split count used; hx_matmul_path 1 = tile kernel, 0 = plain, 2 = the 256x256
 * tile kernel in persistent workgroups (opt-in; the answer for a call without epilogue and with the library's own split). */
int hx_matmul(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
              int64_t ldb_n, int64_t ldc, const void* bias, int bias_dtype, int relu, int in_dtype, int out_dtype,
              int split_k, void* workspace, size_t workspace_bytes, void* stream);
size_t hx_matmul_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                                 int in_dtype, int out_dtype, int has_epilogue, int split_k);
int hx_matmul_splits(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, int in_dtype,
                     int split_k);
int hx_matmul_path(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, int in_dtype,
                   const void* a, const void* b, const void* c, const void* bias);

/* 16-bit attention — the reference's `attention(q, k, v)` (examples/attention.py:33-84): per batch*head
 *   out = cast( (P16 @ v) / l ),  s = (q @ k^T) * (1/sqrt(D) * 1.44269504),  p = exp2(s - rowmax(s)),  l = sum(p),
 * P16 = p cast to the value dtype before the P.V product (:73-74), everything else fp32, softmax evaluated online
 * over key tiles as the reference's compiled kernel does (for 16-bit p the result does not depend on the tiling
 * beyond rounding noise; its eager mode is the one-tile case).
 * scale_dim: the head dimension the softmax scale is taken from, 0 = D (see hx_fp8_attention).
 * q [BH, M, D], k [BH, N, D], v [BH, N, D], out [BH, M, D], contiguous, all of `dtype` (HX_BF16 / HX_F16: MFMA kernel
 * when D is 64 or 128 and the pointers are 16-byte aligned, any M and N; HX_F32 and every other D <= 256: plain
 * kernel).  hx_attention_path: 1 = MFMA kernel, 0 = plain. */
int hx_attention(const void* q, const void* k, const void* v, void* out, int64_t BH, int64_t M, int64_t N, int64_t D,
                 int64_t scale_dim, int dtype, void* stream);
int hx_attention_path(int64_t BH, int64_t M, int64_t N, int64_t D, int dtype, const void* q, const void* k, const void* v,
                      const void* out);

/* ---- Diagnostics (not part of the drop-in interface; no counterpart in the reference) --------------------------------
 * One wave that measures the engine clock of the XCD it lands on as (shader-clock counter delta) / (100 MHz counter
 * delta) over `ticks_100mhz` ticks of the latter (at most 10000 = 100 us; the wave sleeps 3-4 us between two readings of
 * the counter).  out2: device pointer to two uint64 {shader clocks, 100 MHz ticks}; MHz = 100 * out2[0] / out2[1].
 * Launched on a second stream while another kernel runs, it reads the clock that kernel is sustained at, provided that
 * kernel leaves a wave slot free.  Only `bench.py --clock-probe` calls it. */
int hx_clock_probe(uint64_t* out2, int64_t ticks_100mhz, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HX_KERNELS_H */
