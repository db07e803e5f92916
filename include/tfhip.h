/*
 * tfhip.h -- C ABI of libtfhip.so, the MI355X (gfx950) execution runtime behind TensorFrost's
 * backend boundary. Plain pointers and sizes only; no C++ types, no exceptions cross this line.
 *
 * Every function returns TFHIP_OK (0) or a negative status; tfhip_last_error() then holds a
 * human-readable message (HIP / hiprtc error name, compiler log, or the violated precondition).
 * All work is issued on ONE in-order stream owned by the library; only tfhip_d2h, tfhip_sync and
 * tfhip_event_elapsed_ms block the host. Buffers are arrays of 32-bit words, as in the reference
 * (TensorFrost/Backend/CodeGen/Generators.cpp:406-426 -- every kernel argument is uint*).
 */
#ifndef TFHIP_H
#define TFHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TFHIP_OK 0
#define TFHIP_ERR_HIP (-1)      /* a HIP runtime call failed */
#define TFHIP_ERR_COMPILE (-2)  /* hiprtc rejected the source; log in tfhip_last_error() */
#define TFHIP_ERR_ARG (-3)      /* a precondition on the arguments does not hold */
#define TFHIP_ERR_STATE (-4)    /* library not initialised / handle unknown */

typedef struct tfhip_kernel* tfhip_kernel_t;
typedef struct tfhip_event* tfhip_event_t;
typedef struct tfhip_graph* tfhip_graph_t;

/* ---- lifetime -------------------------------------------------------------------------------
 * Replaces the backend start-up arm of InitializeBackend (TensorFrost/Backend/Backend.cpp:49-68,
 * StartOpenGL in Backends/OpenGL/OpenGL.cpp:130-204) and its teardown (Backend.cpp:11-25). */
int tfhip_init(int device);
int tfhip_shutdown(void);
const char* tfhip_last_error(void);
/* Fills name (<= cap bytes), compute-unit count and total HBM bytes of the active device. */
int tfhip_device_info(char* name, size_t cap, int* compute_units, size_t* hbm_bytes);

/* ---- memory ---------------------------------------------------------------------------------
 * Replaces TFCPUBuffer / TFOpenGLBuffer construction, destruction and the two copy virtuals
 * (TensorFrost/Backend/Backends/CPU/Memory.h:18-47, Backends/OpenGL/Memory.h:16-86;
 * interface TensorFrost/Backend/TensorMemory.h:74-88). Sizes and offsets are in 32-bit words. */
int tfhip_malloc(void** dev_ptr, size_t n_words);
int tfhip_free(void* dev_ptr);
int tfhip_h2d(void* dev_dst, size_t dst_offset_words, const uint32_t* host_src, size_t n_words);
int tfhip_d2h(uint32_t* host_dst, const void* dev_src, size_t src_offset_words, size_t n_words); /* blocks */
int tfhip_d2d(void* dev_dst, const void* dev_src, size_t n_words);
int tfhip_fill_u32(void* dev_dst, uint32_t value, size_t n_words);

/* ---- kernels --------------------------------------------------------------------------------
 * Replaces OpenGLKernelManager::createShaderProgram / CompileKernel / DispatchKernel / FreeKernel
 * (TensorFrost/Backend/Backends/OpenGL/KernelManager.h:30-85,105-159,161-166) and the CPU path's
 * dlsym + function-pointer call (Backends/CPU/KernelCompiler.cpp:191-213, CPU/KernelManager.h:28-38).
 *
 * source is HIP C++ holding one `extern "C" __global__` function called kernel_name whose
 * parameters are n_buffers `unsigned*` followed by ONE struct of n_vars 32-bit words (omitted when
 * n_vars == 0). Compiled by hiprtc for gfx950; code objects are cached on disk keyed by a hash of
 * (source, options, hiprtc version) under $TFHIP_CACHE_DIR (default /tmp/tfhip_cache_<uid>, a directory of
 * the calling user); code objects compiled or read once are also kept by the process. */
int tfhip_module_compile(const char* source, const char* kernel_name, const char* options, tfhip_kernel_t* out);
/* Another `extern "C" __global__` function of the module `kernel` was compiled from (same parameter
 * convention). The new handle borrows the module: unload it before, or together with, `kernel`. */
int tfhip_module_get_kernel(tfhip_kernel_t kernel, const char* kernel_name, tfhip_kernel_t* out);
int tfhip_module_unload(tfhip_kernel_t kernel);
/* 1-D grid of grid_x groups of block_x*block_y*block_z threads (the reference always dispatches
 * 1-D over work_group_count: CPP.cpp:503-517, OpenGL/KernelManager.h:141). */
int tfhip_launch(tfhip_kernel_t kernel, uint32_t grid_x, uint32_t block_x, uint32_t block_y, uint32_t block_z,
                 void* const* buffers, size_t n_buffers, const uint32_t* vars, size_t n_vars);
/* Several dispatches of one kernel as ONE launch: grid (grid_x, calls). `kernel` is an entry point whose only parameter is
 * a struct holding an array of per-dispatch arguments (buffer pointers, the variable words, the dispatch's own group
 * count); group (x, y) works on element y and leaves at once when x is beyond that count. `arguments` is that struct,
 * `bytes` long (at most 4096), copied at the call. The reference launches every tf.dispatch on its own (CPP.cpp:482-518,
 * OpenGL/KernelManager.h:105-159); here the kernel manager gathers consecutive small dispatches of the same kernel that
 * touch disjoint buffers, since a launch costs about as much as each of them runs. */
int tfhip_launch_batch(tfhip_kernel_t kernel, uint32_t grid_x, uint32_t calls, uint32_t block_x, const void* arguments, size_t bytes);
/* Replaces Finish() (Backends/OpenGL/OpenGL.cpp:247-249). */
int tfhip_sync(void);
/* Replaces StartDebugRegion / EndDebugRegion behind the Region callback (Backend.cpp:125-133). */
int tfhip_range_push(const char* name);
int tfhip_range_pop(void);

/* ---- timing on the library's stream (no reference counterpart beyond the PROFILE_EXECUTION
 * timer, Backend.cpp:163-177) ---------------------------------------------------------------- */
int tfhip_event_create(tfhip_event_t* out);
int tfhip_event_destroy(tfhip_event_t ev);
int tfhip_event_record(tfhip_event_t ev);
int tfhip_event_elapsed_ms(tfhip_event_t start, tfhip_event_t stop, float* ms); /* blocks on stop */

/* ---- recorded graphs ---------------------------------------------------------------------------
 * Between begin and end every launch, fill and device-to-device copy issued through this library is
 * recorded into a HIP graph instead of running; tfhip_graph_launch then enqueues the whole sequence with
 * one call. This stands in for the per-dispatch host work of a program that is called again and again on
 * the same buffers (Backends/CPU/KernelManager.h:28-38 gathers pointers and calls per dispatch; the emitted
 * TFContext::dispatch builds its argument vectors per dispatch, Backend/CodeGen/Langs/CPP.cpp:482-518).
 * While recording, tfhip_h2d / d2h / sync / free / module_unload are refused, and the scratch buffer of the
 * primitives cannot grow: run the same work once before recording it. tfhip_graph_end(NULL) abandons the
 * recording. A graph refers to the device buffers it was recorded with; they must outlive it.
 * The library's own scratch buffer (partial sums, look-back status words, sort histograms) is part of that rule and
 * the library keeps it: while any graph is alive, a scratch buffer that must grow for later eager work is parked, not
 * freed, and released when the last graph is destroyed. */
int tfhip_graph_begin(void);
int tfhip_graph_end(tfhip_graph_t* out);
int tfhip_graph_node_count(tfhip_graph_t graph, size_t* nodes);
int tfhip_graph_launch(tfhip_graph_t graph);
int tfhip_graph_destroy(tfhip_graph_t graph); /* waits for the stream first */

/* ---- introspection (no reference counterpart; used by the tests of the bookkeeping above) ----------------------
 * Size of the scratch buffer of the primitives, how many outgrown scratch buffers are parked because recorded graphs
 * may still point into them, and how many graphs are alive. */
int tfhip_scratch_info(size_t* bytes, size_t* retired_buffers, size_t* live_graphs);
/* Grows the scratch buffer to at least `bytes`, as a primitive with that need would. */
int tfhip_scratch_reserve(size_t bytes);
/* The two hooks that let the error paths be tested without any kernel misbehaving are declared in tfhip_test.h. */

/* ---- data-parallel primitives ---------------------------------------------------------------
 * The reference lowers these to one-thread-per-output serial loops inside generated kernels
 * (TensorFrost/Compiler/Implementations.cpp:243-303 reduction, :305-359 scan, :560-646 matmul;
 * two-stage split of long axes Compiler/Steps/Optimization.cpp:469-510). The emitter recognises
 * those loops and dispatches here instead. All matrices are dense row-major fp32/u32 words. */

#define TFHIP_REDUCE_SUM 0
#define TFHIP_REDUCE_MAX 1
#define TFHIP_REDUCE_MIN 2

/* out[r] = op_c x[r*cols + c]; rows, cols >= 1. Initial values as Implementations.cpp:374-426
 * (0, -FLT_MAX, +FLT_MAX). */
int tfhip_reduce_rows_f32(int op, const float* x, float* out, size_t rows, size_t cols);
int tfhip_reduce_sum_f32_rows(const float* x, float* out, size_t rows, size_t cols);
int tfhip_reduce_max_f32_rows(const float* x, float* out, size_t rows, size_t cols);
int tfhip_reduce_min_f32_rows(const float* x, float* out, size_t rows, size_t cols);
/* out[c] = op_r x[r*cols + c] (the strided case). */
int tfhip_reduce_cols_f32(int op, const float* x, float* out, size_t rows, size_t cols);
/* out[s*cols + c] = op over rows [s*rows_per_slab, (s+1)*rows_per_slab) of column c (the last slab may be short):
 * the first stage of an axis-0 reduction that OptimizeReductions has split into chunks of 128
 * (Compiler/Steps/Optimization.cpp:469-510), as one launch. */
int tfhip_reduce_cols_slabs_f32(int op, const float* x, float* out, size_t rows, size_t cols, size_t rows_per_slab);
int tfhip_reduce_sum_f32_cols(const float* x, float* out, size_t rows, size_t cols);
int tfhip_reduce_max_f32_cols(const float* x, float* out, size_t rows, size_t cols);
int tfhip_reduce_min_f32_cols(const float* x, float* out, size_t rows, size_t cols);

/* y[r,c] = exp(x[r,c] - max_c x[r,:]) / sum_c exp(x[r,c] - max_c x[r,:]); one read and one write of
 * the matrix. The reference builds this from >= 5 generated kernels (user-level composition, e.g.
 * tests/autograd_test.py:29-31, examples/ML/MNIST/module.py:8-10). x == y (in place) is allowed. */
int tfhip_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols);
/* The same, and the two per-row intermediates of that composition as well: row_max[r] = max_c x[r,:] (what the
 * reference's max kernels leave in their output tensor, Implementations.cpp:243-303) and row_sum[r] =
 * sum_c exp(x[r,c] - row_max[r]) (the sum kernels' output). The kernel manager calls this when a program dispatches
 * that whole chain of kernels, because the program may still read the two tensors afterwards. y may be null: then only
 * the two statistics are computed, from one read of x (what a log-softmax needs: (x - max) - log(sum)). */
int tfhip_softmax_rows_stats_f32(const float* x, float* y, float* row_max, float* row_sum, size_t rows, size_t cols);
/* Row log-softmax, y[r,c] = (x[r,c] - max_c x[r,:]) - log(sum_c exp(x[r,c] - max)), as the reference's own tests compose
 * it (tests/autograd_test.py:29-31: the max and sum kernels of the softmax, then one element-wise kernel): one read and
 * one write of the matrix, the same kernels and row-length cases as the softmax. The second form also leaves the two
 * per-row intermediates, as tfhip_softmax_rows_stats_f32 does; the kernel manager calls it when a program dispatches
 * that chain of kernels. */
int tfhip_log_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols);
int tfhip_log_softmax_rows_stats_f32(const float* x, float* y, float* row_max, float* row_sum, size_t rows, size_t cols);

/* out[i] = x[0] + ... + x[i] over a contiguous array; in == out is allowed; n == 0 is a no-op.
 * Replaces the one-thread serial loop of dim_prefix_sum (Implementations.cpp:305-359,447-449).
 * u32/i32 wrap modulo 2^32 exactly as the C++ loop does (bit-exact); f32 sums in a fixed tiled order
 * (reproducible run to run, within 1e-4 relative of the serial order). */
int tfhip_scan_inclusive_u32(const uint32_t* x, uint32_t* out, size_t n);
int tfhip_scan_inclusive_i32(const int32_t* x, int32_t* out, size_t n);
int tfhip_scan_inclusive_f32(const float* x, float* out, size_t n);
/* tfhip_scan_inclusive_u32 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same result, bit for bit; the ticket and the
 * per-tile status words of the look-back live in a fixed 512 KiB array in device memory that every GPU the library runs on
 * holds until the process ends, located once by tfhip_init. It calls no hipMalloc / hipFree and no allocating library
 * routine; n above 2^30 elements is refused with TFHIP_ERR_ARG. All calls on one GPU share that array (each call clears
 * the words it needs with a fill kernel first): calls that overlap in time on one GPU race, so issue them on the
 * library's one stream, as every call here is. x == out is allowed; n == 0 is a no-op. */
int tfhip_scan_inclusive_u32_static(const uint32_t* x, uint32_t* out, size_t n);
/* The same along the last axis of a row-major [rows, cols] matrix: out[r, i] = x[r, 0] + ... + x[r, i], every row on
 * its own (the kernel shape of dim_prefix_sum over the last axis: one thread per row in the reference). u32 serves
 * i32 as well (wrap-around is the same). */
int tfhip_scan_inclusive_rows_u32(const uint32_t* x, uint32_t* out, size_t rows, size_t cols);
int tfhip_scan_inclusive_rows_f32(const float* x, float* out, size_t rows, size_t cols);
/* Down the columns of `batch` row-major matrices [rows, cols] that follow each other: out[b, r, c] = x[b, 0, c] + ... +
 * x[b, r, c] (dim_prefix_sum over an axis that is not the last: one thread per (b, c) walking r in the reference; the
 * radix sort scans its [groups, 64] histograms this way, Python/TensorFrost/sort.py:39-50). */
int tfhip_scan_inclusive_cols_u32(const uint32_t* x, uint32_t* out, size_t batch, size_t rows, size_t cols);
int tfhip_scan_inclusive_cols_f32(const float* x, float* out, size_t batch, size_t rows, size_t cols);

#define TFHIP_KEY_U32 0
#define TFHIP_KEY_I32 1
#define TFHIP_KEY_F32 2
/* Or-ed to TFHIP_KEY_I32 / TFHIP_KEY_F32: keys_in holds int / float keys, keys_out receives their order-preserving
 * unsigned images (sort.py:54-60,68-69) in sorted order, i.e. what the reference's `Radix sort` region leaves in its
 * key buffer before map_uint_to_float / map_uint_to_int run (sort.py:178-182). */
#define TFHIP_KEY_KEEP_MAPPED 0x100

/* Stable ascending sort of n 32-bit keys with an optional 32-bit payload (vals_in == vals_out == NULL
 * sorts keys only). Replaces the whole `Radix sort` region that tf.sort.radix emits
 * (Python/TensorFrost/sort.py:38-187: 6 passes x ~7 generated kernels) with 2 + 4 launches.
 * Out of place: keys_in/vals_in are not modified and must differ from keys_out/vals_out.
 * keys_tmp/vals_tmp are n-word ping-pong buffers (the reference's keys1/values1, sort.py:96-100);
 * pass NULL to let the library use its own scratch. n == 0 is a no-op; n < 2^30.
 * key_kind selects the order-preserving key mapping of sort.py:52-72 (i32: flip the sign bit; f32: flip
 * all bits of negatives, the sign bit otherwise; so -0.0 sorts before +0.0 and NaNs by bit pattern). */
int tfhip_radix_sort_kv(int key_kind, const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out, uint32_t* vals_out,
                        uint32_t* keys_tmp, uint32_t* vals_tmp, size_t n);
int tfhip_radix_sort_kv_u32(const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out, uint32_t* vals_out,
                            uint32_t* keys_tmp, uint32_t* vals_tmp, size_t n);

/* C[M,N] = op(A) * op(B) in fp32 on the matrix cores (fp32 inputs, fp32 accumulation), dense row-major:
 *   nn: A[M,K] B[K,N]      nt: A[M,K] B[N,K]      tn: A[K,M] B[K,N]
 * Replaces the one-thread-per-element serial-k loop of tf.matmul (Implementations.cpp:560-646) and the two
 * transposed products of its backward pass (:133-135, transposes fused as index remaps :451-488).
 * C must not overlap A or B. K == 0 gives C = 0. */
int tfhip_sgemm_nn(const float* A, const float* B, float* C, size_t M, size_t N, size_t K);
int tfhip_sgemm_nt(const float* A, const float* B, float* C, size_t M, size_t N, size_t K);
int tfhip_sgemm_tn(const float* A, const float* B, float* C, size_t M, size_t N, size_t K);
/* The weight gradient and the bias gradient of a dense layer from one read of the upstream gradient: C = A^T B as
 * tfhip_sgemm_tn (A[K,M] the layer's input, B[K,N] = dY), and colsum_b[n] = sum_k B[k,n]. In the reference these are
 * two kernels that both read dY: the matmul loop of the backward pass (Implementations.cpp:133-135,560-646) and the
 * dim_sum over axis 0 that the broadcast bias's gradient lowers to (:243-303). For M >= 128 the sums ride in the tiled
 * product (the groups of the first tile row add up the panels of B they stage), for narrow results with a long K in the
 * kernel that feeds both operands straight from memory; other shapes run the product's own best kernel and a column
 * reduction. C is bit-identical to tfhip_sgemm_tn's. */
int tfhip_sgemm_tn_colsum(const float* A, const float* B, float* C, float* colsum_b, size_t M, size_t N, size_t K);

/* The same products with the element-wise tail that TensorFrost's kernel fusion leaves behind the matmul loop
 * of a dense layer (the loop of Implementations.cpp:560-646 followed, in the same kernel, by the bias add and
 * activation of e.g. examples/ML/MNIST/module.py, or by the ReLU mask of its backward pass), applied to each
 * element of the product on its way to C:
 *   TFHIP_EPILOGUE_BIAS           C[m,n] = P[m,n] + aux[n]
 *   TFHIP_EPILOGUE_BIAS_RELU      C[m,n] = max(P[m,n] + aux[n], 0)
 *   TFHIP_EPILOGUE_MASK_POSITIVE  C[m,n] = aux[m,n] > 0 ? P[m,n] : 0      (aux dense [M,N])
 * aux must not overlap C. */
#define TFHIP_GEMM_NN 0
#define TFHIP_GEMM_NT 1
#define TFHIP_GEMM_TN 2
#define TFHIP_EPILOGUE_NONE 0
#define TFHIP_EPILOGUE_BIAS_RELU 1
#define TFHIP_EPILOGUE_BIAS 2
#define TFHIP_EPILOGUE_MASK_POSITIVE 3
int tfhip_sgemm_fused(int layout, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, int epilogue, const float* aux);
/* `batch` products in one launch: matrix t of an operand starts stride_* elements after matrix t - 1 (stride 0: the
 * operand is shared by the whole batch). The reference's matmul carries leading batch dimensions through its loop
 * (Compiler/Implementations.cpp:575-633, indices_c[2..] appended to the indices of A and B, broadcast where an
 * operand has fewer dimensions). At most 65535 products per call; results must not overlap. */
int tfhip_sgemm_batched(int layout, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, size_t batch, size_t stride_a, size_t stride_b,
                        size_t stride_c);

#ifdef __cplusplus
}
#endif
#endif /* TFHIP_H */
