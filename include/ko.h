/*
 * ko.h - C ABI of the gfx950 (MI355X) operator library libko.so.
 *
 * Plain C: no HIP types, no C++ types.  Pointers named `in`, `out`, `A`, ...
 * are DEVICE pointers unless the comment says host.  A stream is an opaque
 * handle (a hipStream_t underneath; NULL is the default stream).  Every
 * function returns a ko_status; 0 is success.  ko_last_error_string() returns
 * a thread-local description of the last failure on the calling thread.
 *
 * The reference (donglinz/kernel_optimization) has no FFI: its seam is the
 * `Tensor` class plus three `__global__` templates launched with
 * <<<grid, block, smem, stream>>>.  Each entry point below names the reference
 * interface it stands in for.
 */
#ifndef KO_H
#define KO_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ko_stream_t;
typedef void *ko_event_t;

typedef enum ko_status {
    KO_OK = 0,
    KO_ERR_INVALID_ARGUMENT = 1,  /* null pointer, negative size, bad enum */
    KO_ERR_UNSUPPORTED_SHAPE = 2, /* e.g. a row longer than the chosen policy holds */
    KO_ERR_RUNTIME = 3,           /* a HIP runtime call or a kernel launch failed */
    KO_ERR_OUT_OF_MEMORY = 4,
    KO_ERR_NO_DEVICE = 5
} ko_status;

/* Row-mapping policy: the reference's three implementations per operator.
 * WARP  = row per (sub-)wavefront, row held in registers
 *         (SoftMaxWarpImpl softmax.h:11-60, LayerNormWarpImpl layernorm.h:145-201)
 * BLOCK = row per workgroup, row held on chip, LDS only for cross-wave partials
 *         (SoftMaxBlockImpl softmax.h:62-113, LayerNormBlockImpl layernorm.h:204-252)
 * BLOCK_NOCACHE = row per workgroup, row re-read from global memory
 *         (SoftMaxBlockNoCacheImpl softmax.h:116-166, LayerNormBlockNoCacheImpl layernorm.h:254-300)
 * AUTO  = chosen from the row length: the first of the three that holds the row.
 * Longest rows: WARP 2048 fp32 / 4096 16-bit columns; BLOCK softmax 135168 fp32 / 172032 16-bit columns
 * (98304 columns with a padding mask), LayerNorm any length (what the chip does not hold is read twice);
 * BLOCK_NOCACHE any length.  Rows that are walked element by element (a row length that is not a whole number of
 * 16-byte vectors, or tensors off 16-byte boundaries): WARP 2048 columns, BLOCK softmax 65536 columns, LayerNorm
 * any length.  A policy asked for explicitly runs that policy's kernel; on a longer row than it holds it returns
 * KO_ERR_UNSUPPORTED_SHAPE. */
typedef enum ko_policy {
    KO_POLICY_AUTO = 0,
    KO_POLICY_WARP = 1,
    KO_POLICY_BLOCK = 2,
    KO_POLICY_BLOCK_NOCACHE = 3
} ko_policy;

typedef enum ko_dtype16 { KO_F16 = 0, KO_BF16 = 1 } ko_dtype16;

/* Epilogue activations of the 16-bit GEMM: GELU(x) = x/2 (1 + erf(x / sqrt 2)), or its tanh form
 * x/2 (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))). */
typedef enum ko_activation { KO_ACT_NONE = 0, KO_ACT_GELU_ERF = 1, KO_ACT_GELU_TANH = 2 } ko_activation;
typedef enum ko_layout { KO_ROW_MAJOR = 0, KO_COL_MAJOR = 1 } ko_layout;

typedef struct ko_device_info_t {
    char name[256];
    char arch[64];              /* "gfx950..." */
    int compute_units;
    int wavefront_size;
    int clock_khz;              /* peak engine clock */
    int memory_clock_khz;
    int memory_bus_bits;
    int l2_bytes;
    int lds_bytes_per_workgroup;
    size_t hbm_bytes;
} ko_device_info_t;

/* ---- runtime: replaces the CUDA runtime calls made by common/tensor.cu:8-42,
 *      checkCudaErrors (common/common.h:16-25) and the stream/event calls of the
 *      benchmark drivers (nn_operators/softmax/main.cu:28-29,44-68). ---------- */
const char *ko_last_error_string(void);
const char *ko_status_name(int status);
int ko_device_info(ko_device_info_t *info);

int ko_malloc(void **device_ptr, size_t bytes);                 /* cudaMalloc, tensor.cu:10 */
int ko_free(void *device_ptr);                                  /* cudaFree,   tensor.cu:25 */
int ko_memset_async(void *device_ptr, int value, size_t bytes, ko_stream_t stream);
int ko_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes);                            /* tensor.cu:28-30 */
int ko_memcpy_h2d_async(void *device_dst, const void *host_src, size_t bytes, ko_stream_t stream);  /* tensor.cu:32-34 */
int ko_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes);                            /* tensor.cu:36-38 */
int ko_memcpy_d2h_async(void *host_dst, const void *device_src, size_t bytes, ko_stream_t stream);  /* tensor.cu:40-42 */
int ko_memcpy_d2d_async(void *device_dst, const void *device_src, size_t bytes, ko_stream_t stream);

int ko_stream_create(ko_stream_t *stream);       /* cudaStreamCreateWithFlags(NonBlocking), softmax/main.cu:29 */
int ko_stream_destroy(ko_stream_t stream);        /* waits for the stream's work, frees its workspace (see ko_sgemm_f32) */
int ko_stream_synchronize(ko_stream_t stream);   /* softmax/main.cu:46,70 */
int ko_device_synchronize(void);                 /* gemm/main.cu:152 */

int ko_event_create(ko_event_t *event);                             /* softmax/main.cu:49-50 */
int ko_event_record(ko_event_t event, ko_stream_t stream);          /* softmax/main.cu:57,61 */
int ko_event_synchronize(ko_event_t event);                         /* softmax/main.cu:63 */
int ko_event_elapsed_ms(float *ms, ko_event_t start, ko_event_t stop); /* softmax/main.cu:66 */
int ko_event_destroy(ko_event_t event);

/* ---- row softmax: replaces
 *      softmax<K><<<grid, block, K::smem_in_bytes, stream>>>(T *in, T *out)
 *      (nn_operators/softmax/softmax.h:168-174, launched at softmax/main.cu:58-60).
 * in, out: row-major [rows, cols] fp32, contiguous; in == out is allowed.  Tensors that start on 16-byte
 * boundaries are the fast case; any 4-byte aligned address is accepted (walked element by element, see cols).
 * Any cols: a multiple of 4 (one 16-byte vector: the reference's vec_len = 4, softmax.h:21) is the fast case;
 * other row lengths start their rows off 16-byte boundaries and are walked element by element (what the
 * reference's descriptors do with vec_len = 1 or 2), at 0.6-0.9 of the rate.
 * valid_len: NULL for no mask, else device int32[ceil(rows / rows_per_seq)];
 * row r belongs to sequence r / rows_per_seq and every column
 * j >= valid_len[seq] takes the value -10000 before the softmax.
 * Workspace: a few long rows (fewer rows than a quarter of the compute units, 256 KB and more each) run as two
 * launches that pass partial results through 1 MiB of device memory that belongs to the (device, stream) pair -
 * an allocation of its own next to the GEMMs' workspace described at ko_sgemm_f32, made at the first such call,
 * kept and released the same way, under the same rules for graphs; the same holds for ko_layernorm_f32 and the
 * 16-bit forms.  Without a workspace (first such call inside a graph capture)
 * they run as one launch, one workgroup per row. */
int ko_softmax_f32(const float *in, float *out, int64_t rows, int64_t cols,
                   const int32_t *valid_len, int64_t rows_per_seq, ko_stream_t stream);

/* Same with the policy fixed by the caller (the three descriptor types). */
int ko_softmax_f32_policy(const float *in, float *out, int64_t rows, int64_t cols,
                          const int32_t *valid_len, int64_t rows_per_seq, int policy,
                          ko_stream_t stream);

/* Same operator on 16-bit storage: in, out are binary16 (KO_F16) or bfloat16 (KO_BF16) bit
 * patterns, the arithmetic is fp32, the result is rounded once to the storage type.  cols that are
 * a multiple of 8 (one 16-byte vector) are the fast case, other lengths as for fp32.  Stands in for the reference's T = half instantiation
 * of the same template (softmax.h:11, with the half functors of common/functors.h:71-77 and
 * limits of common/common.h:171-177).  policy: a ko_policy value. */
int ko_softmax_16(const void *in, void *out, int64_t rows, int64_t cols, const int32_t *valid_len,
                  int64_t rows_per_seq, int dtype, int policy, ko_stream_t stream);

/* ---- LayerNorm: replaces
 *      layer_normalization<K><<<...>>>(Element *in, Element *out, Element epsilon,
 *                                      Element *gamma = nullptr, Element *beta = nullptr)
 *      (nn_operators/layernorm/layernorm.h:302-312, launched at layernorm/main.cu:57-59).
 * in, out: row-major [rows, cols] fp32 (in == out allowed); gamma, beta: [cols]
 * or NULL (each independently); mean, rstd: [rows] outputs or NULL.
 * var divides by cols (unbiased == 0) or cols - 1 (unbiased != 0, the
 * reference's intent at layernorm.h:48).  Any cols; multiples of 4 are the fast case (see ko_softmax_f32). */
int ko_layernorm_f32(const float *in, float *out, float *mean, float *rstd, const float *gamma,
                     const float *beta, int64_t rows, int64_t cols, float eps, int unbiased,
                     ko_stream_t stream);

int ko_layernorm_f32_policy(const float *in, float *out, float *mean, float *rstd,
                            const float *gamma, const float *beta, int64_t rows, int64_t cols,
                            float eps, int unbiased, int policy, ko_stream_t stream);

/* Same operator on 16-bit storage: in, out, gamma, beta are binary16 or bfloat16 bit patterns
 * (all of the one dtype), mean and rstd stay fp32, the arithmetic is fp32.  Any cols; multiples
 * of 8 are the fast case.  Stands in for Element = half in LayerNormWarpImpl and its siblings
 * (layernorm.h:145, with Rsqrt<half> of common/functors.h:105-111). */
int ko_layernorm_16(const void *in, void *out, float *mean, float *rstd, const void *gamma,
                    const void *beta, int64_t rows, int64_t cols, float eps, int unbiased, int dtype,
                    int policy, ko_stream_t stream);

/* ---- SIMT-path SGEMM: replaces
 *      gemm<GemmKernelSimt<...>><<<grid, K::thread_per_block, K::smem_total_size_in_bytes, stream>>>
 *          (shape::GemmCoord problem_size, ElementA *A, ElementB *B, ElementC *C, ElementC *D)
 *      (nn_operators/gemm/gemm.h:11-21, simt_gemm.h:299-374, launched at gemm/main.cu:111-117).
 * D[m,n] = alpha * A[m,k] * B[k,n] + beta * C[m,n], all row-major fp32.
 * C may be NULL (then beta is ignored); the reference's epilogue is alpha = beta = 1
 * with C given, or D = A*B with C null (simt_gemm.h:325-373).
 * m, n, k multiples of 4 and 16-byte aligned pointers are not required (operand rows that do not start on
 * 16-byte boundaries are loaded four bytes at a time: about 0.7 of the aligned rate); any positive sizes are
 * accepted.  m == 0 or n == 0 is a no-op; k == 0 is the empty product, D = beta * C (zero without a C) in one
 * scale-and-copy launch, as the reference's kernel leaves it when its main loop runs no K tile
 * (simt_gemm.h:325-354); A and B may be NULL then.  The 16-bit entries do the same: D = activation(beta * C + bias).
 * Workspace: a problem with a deep K whose output tiles do not fill the chip (tiles for at most half of the
 * compute units and k >= 768, or rounds of tiles that leave many compute units idle and k >= 2048; any n)
 * is cut into slices of K that run side by side; their partial products go
 * through the first 32 MiB of a 64 MiB block of device memory that the library allocates at the first such call
 * on a (device, stream) pair and keeps until ko_stream_destroy releases it (the default stream's: until the process ends).  Calls on
 * different streams therefore never share it.  A first such call made while the stream is being captured into a
 * graph allocates nothing and takes the unsliced kernels; so does every call while 64 live pairs hold a
 * workspace.  Results do not depend on the timing of the slices (summed in slice order), but the sliced and the
 * unsliced path round differently.
 * Graphs: a sliced call captured on a stream that already has its workspace records that workspace's address.
 * Replay such a graph only in stream order with the other work of the stream it was captured on (a replay on
 * another stream, or two replays in flight at once, race on the workspace with each other and with eager
 * sliced calls on the origin stream and give wrong sums), and not after that stream was destroyed (its
 * workspace is freed then).  ko_sgemm_f32_static_scratch is the entry for graphs that must not depend on a
 * stream's lifetime. */
int ko_sgemm_f32(int64_t m, int64_t n, int64_t k, float alpha, const float *A, const float *B,
                 float beta, const float *C, float *D, ko_stream_t stream);

/* The same operator for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments,
 * same kernels and the same bits as ko_sgemm_f32, but the partial products of a K-sliced problem go to an
 * 32 MiB array that is part of the library's device code (one copy per GPU, held until the process ends)
 * instead of a workspace allocated for the stream: the call makes no hipMalloc or hipFree, also not the
 * first one on a stream.  A slice plan whose partial products exceed the array is refused with
 * KO_ERR_UNSUPPORTED_SHAPE (plans chosen by shape are chosen to fit; only a slice count forced through the
 * harness's tuning knob "sgemm.k_slices" can exceed it).
 * All calls on one GPU share the array: calls that overlap in time on one GPU (different streams, different
 * threads) race on it and must be serialised by the caller.  Nothing in it has to start at zero: every
 * element the summing kernel reads was written by the same call.  The first call on a device looks up the
 * array's address (no stream work; make it outside a capture). */
int ko_sgemm_f32_static_scratch(int64_t m, int64_t n, int64_t k, float alpha, const float *A, const float *B,
                                float beta, const float *C, float *D, ko_stream_t stream);

/* ---- tensor-core-path GEMM: replaces
 *      gemm<GemmKernelTensorCore<half, half, half, ...>><<<...>>>(problem_size, A, B, C, D)
 *      (nn_operators/gemm/tensor_core_gemm.h:341-399; its launch is commented out at gemm/main.cu:344).
 * A [m,k] row-major; B logical [k,n], stored row-major (b_layout = KO_ROW_MAJOR,
 * the reference's layout, tensor_core_gemm.h:178) or column-major (KO_COL_MAJOR:
 * memory [n][k]); C, D [m,n] row-major.  Elements are binary16 or bfloat16
 * (in_dtype); products accumulate in fp32 on the matrix cores; D is rounded once
 * to the 16-bit type.  C may be NULL.  k must be a multiple of 8; A, B, C, D 16-byte aligned.
 * m and n are free: an n that is not a multiple of 8 (rows of C and D off 16-byte boundaries) keeps the fast
 * kernels with a column-major B and costs about a tenth; with a row-major B (whose own rows are off 16-byte
 * boundaries then) it runs at about 0.6 of the rate.
 * Workspace: like ko_sgemm_f32, a deep K (k >= 2048; k >= 1536 on very few tiles; any n) on few output tiles -
 * of the whole problem or of the parts a ragged shape is cut into - is cut into slices of K whose fp32
 * partial products go through the 64 MiB workspace of the (device, stream) pair, allocated at the first such
 * call on the stream; a first such call inside a graph capture allocates nothing and runs unsliced.  Beyond k = 8192
 * that also holds for outputs of up to half a chip's worth of 256 x 256 tiles (n a multiple of 256). */
int ko_gemm_f16f32acc(int64_t m, int64_t n, int64_t k, float alpha, const void *A, const void *B,
                      int b_layout, float beta, const void *C, void *D, int in_dtype,
                      ko_stream_t stream);

/* Same with the rest of a feed-forward up-projection fused into the epilogue:
 *      D = activation(alpha * A B + beta * C + bias),   bias: [n] in the 16-bit type or NULL,
 * evaluated in fp32 and rounded once.  The reference's epilogue is D = acc + C
 * (simt_gemm.h:325-354; the tensor-core one is unfinished, tensor_core_gemm.h:366-397) and its
 * functor header carries MultiplyAdd for such fusions (common/functors.h); the 16384 x 3072 x 768
 * configuration is that projection's shape.  activation: a ko_activation value. */
int ko_gemm_f16f32acc_bias_act(int64_t m, int64_t n, int64_t k, float alpha, const void *A,
                               const void *B, int b_layout, float beta, const void *C,
                               const void *bias, int activation, void *D, int in_dtype,
                               ko_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KO_H */
