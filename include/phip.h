/*
 * libphip: C ABI of the MI355X (gfx950) backend for primitiv's matmul path.
 *
 * Everything primitiv's `devices::HIP` class needs from the GPU goes through
 * these entry points: plain pointers and sizes, an int status, no C++ types.
 * Each declaration names the interface of the reference (primitiv v0.4.0,
 * paths relative to its root) that it stands behind.
 *
 * Conventions
 *  - Every function returns PHIP_OK (0) or a negative PHIP_ERR_* code and
 *    never throws.  phip_last_error() returns the calling thread's message
 *    for the most recent failure.
 *  - Device pointers are raw HIP device addresses.  Matrices are dense
 *    column-major (leading dimension = rows); the minibatch is the outermost
 *    index with stride rows*cols, or stride 0 for an operand whose batch is 1
 *    (primitiv/devices/eigen/ops/matmul.cc:18-37).
 *  - All device work of a context is enqueued in order on that context's one
 *    stream; only the *_d2h copies, phip_sync and phip_event_elapsed_ms block
 *    the host.  In-order execution is what makes immediate reuse of a pool
 *    block safe (the reference relies on the same property of the CUDA null
 *    stream, primitiv/devices/cuda/ops/copy_tensor.cu:20-23).
 *  - A context is driven by one host thread at a time, like a device object of
 *    the reference (its devices keep unguarded per-object state too, e.g.
 *    primitiv/devices/cuda/device.h:242-248); different contexts may be used
 *    from different threads.  Only the pool entry points (phip_pool_alloc,
 *    phip_pool_free, phip_pool_free_by_id, phip_pool_stats) take the context's
 *    lock, because tensor handles may be released from any thread.
 *  - Element types: f32 = float, f16 = IEEE binary16, bf16 = bfloat16.  The
 *    16-bit variants store 16-bit values and always accumulate in fp32.
 */
#ifndef PHIP_H_
#define PHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PHIP_OK 0
#define PHIP_ERR_INVALID_ARGUMENT (-1)
#define PHIP_ERR_RUNTIME (-2)        /* a HIP runtime call failed */
#define PHIP_ERR_OUT_OF_MEMORY (-3)
#define PHIP_ERR_UNSUPPORTED (-4)    /* device is not a gfx950 part, etc. */

typedef struct phip_ctx phip_ctx;
typedef struct phip_event phip_event;
typedef struct phip_randomizer phip_randomizer;

typedef struct phip_device_info {
  char name[256];
  char arch[64];             /* e.g. "gfx950:sramecc+:xnack-" */
  int32_t device_id;
  int32_t compute_units;
  int32_t clock_mhz;         /* peak engine clock */
  int32_t memory_clock_mhz;
  int32_t memory_bus_bits;
  int32_t wavefront_size;
  int32_t lds_bytes_per_workgroup;
  int32_t l2_bytes;
  uint64_t global_memory_bytes;
} phip_device_info;

/* ---- errors --------------------------------------------------------------
 * Reference: exceptions `primitiv::Error` raised through PRIMITIV_THROW_ERROR
 * (primitiv/core/error.h:14-60) and CUDA_CALL (primitiv/internal/cuda/utils.h:
 * 20-28); the host class turns a non-zero status plus this message into that
 * exception. */
const char *phip_last_error(void);

/* ---- devices and contexts -------------------------------------------------
 * Reference: CUDA::num_devices / assert_support / check_support / ctor / dtor
 * (primitiv/devices/cuda/device.cu:12-116, primitiv/devices/cuda/device.h:
 * 27-62) and cuda::InternalState (primitiv/internal/cuda/utils.h:320-350). */
int phip_device_count(int *count);
/* PHIP_OK when `device_id` exists, is a gfx950 part and has >= 1 GiB. */
int phip_check_support(int device_id);
int phip_ctx_create(int device_id, phip_ctx **out);
/* Frees every pool block, the stream and the context. */
int phip_ctx_destroy(phip_ctx *ctx);
/* Process-unique id of a live context (never reused); 0 is never an id. */
uint64_t phip_ctx_id(const phip_ctx *ctx);
int phip_device_info_get(phip_ctx *ctx, phip_device_info *out);
/* Writes the human-readable description used by Device::dump_description
 * (primitiv/devices/cuda/ops/dump_description.cu:12-40) into buf. */
int phip_describe(phip_ctx *ctx, char *buf, size_t buf_size);
int phip_sync(phip_ctx *ctx);
/* Bit-reproducible gradients.  No counterpart in the reference's interface: its
 * CPU devices add in one fixed order by construction, its CUDA device does not
 * (atomicAdd, e.g. primitiv/devices/cuda/ops/add.cu:16-27).  By default a
 * matmul_bw product whose contraction is cut between workgroups adds its tiles
 * into the accumulated gradient with fp32 atomics: every run is right to
 * rounding (about 1e-7 relative), the bits depend on the order of arrival.
 * With on != 0 such products exchange fp32 partial tiles instead and the last
 * workgroup of a tile adds them in a fixed order, as forward products always
 * do: the same bits on every run, at the cost of one more round trip through
 * memory per launch (and the two gradient products no longer share a launch). */
int phip_set_deterministic(phip_ctx *ctx, int on);
/* Two lanes for matrix products.  No counterpart in the reference's interface
 * (its CUDA device enqueues everything on one stream).  A context runs matmul
 * calls that follow one another and do not touch each other's operands on two
 * streams at once - per-timestep products leave most of the GPU idle for most
 * of their launch - and keeps what the caller observes in the order of its
 * calls: a product waits for every earlier one whose operands it overlaps in
 * memory, and every other operation (elementwise work, copies, phip_sync,
 * phip_event_record) waits for both lanes.  The second stream comes into use
 * with the sixth such call in a row and goes out of use with the first
 * operation of another kind that enqueues work; a fill (phip_fill_*) counts
 * as a matmul call here (a backward pass resets every gradient before it adds
 * products into it).  Products of more than 4 GFLOP and allocation-free calls
 * always run in order.  on == 0 puts every launch back
 * on one stream; the environment variable PHIP_OVERLAP=0 makes that the
 * default of contexts created afterwards.  The call itself waits for neither
 * lane on the host. */
int phip_set_overlap(phip_ctx *ctx, int on);
/* Zero fills that are only noted.  No counterpart in the reference's interface.
 * primitiv's backward pass gives every gradient a zero-filled tensor and then
 * calls an operator that adds into it (primitiv/core/graph.cc:192-216) - two
 * launches per gradient where the tensors are small and a launch costs more
 * than its work.  By default phip_fill_* with the value +0 launches nothing:
 * the range is noted, and the next entry point of the context either is a
 * gradient operation (phip_unary_bw_*, phip_const_bw_*, phip_pown_bw_*,
 * phip_binary_bw_*, phip_inplace_add_*, phip_inplace_subtract_*) whose output
 * is exactly that range - it then writes 0 + value instead of reading and
 * adding, the same bits - or launches the noted fills first, in the order they
 * were asked for.  Nothing the caller can observe changes: every entry point
 * that reads, writes, copies or waits sees the memory as if the fill had run
 * when it was called, and a block handed back with phip_pool_free simply
 * forgets its fill.  Memory that the caller touches behind the library's back
 * (its own HIP calls on the raw pointers) would see the difference; on == 0
 * launches every fill at once, as does the environment variable
 * PHIP_DEFER_ZERO_FILLS=0 for contexts created afterwards. */
int phip_set_deferred_zero_fill(phip_ctx *ctx, int on);

/* ---- raw memory -----------------------------------------------------------
 * Reference: the allocator / deleter lambdas handed to MemoryPool
 * (primitiv/internal/cuda/utils.h:330-340).  phip_malloc fails with
 * PHIP_ERR_OUT_OF_MEMORY so the caller's pool can release blocks and retry
 * (primitiv/core/memory_pool.cc:53-63).  Before it gives up, phip_malloc
 * frees the idle blocks of the pooled memory below (every context on the same
 * GPU) and tries once more. */
int phip_malloc(phip_ctx *ctx, size_t bytes, void **out);
int phip_free(phip_ctx *ctx, void *ptr);

/* ---- pooled memory --------------------------------------------------------
 * Reference: MemoryPool::allocate / free / release_reserved_blocks
 * (primitiv/core/memory_pool.cc:35-95): request rounded up to a power of two
 * (at least `2*sizeof(float)`, primitiv/internal/cuda/utils.h:337-342),
 * per-size free lists, one retry after releasing the reserved blocks.
 * bytes == 0 yields *out = NULL, *allocated = 0.  The library takes the scratch
 * memory of its elementwise, reduction and convolution kernels from the same
 * pool (unfolded images, partial reductions, index lists); the scratch of the
 * matrix products (partial tiles of split products, a transposed 16-bit
 * operand) comes from a second pool of the same policy whose blocks are never
 * handed to a caller, because products may run on two streams (see
 * phip_set_overlap) and a block is reused in stream order.  Blocks of both
 * are powers of two and stay cached until released; the retry releases the
 * idle blocks of every context on the GPU. */
int phip_pool_alloc(phip_ctx *ctx, size_t bytes, void **out, size_t *allocated);
int phip_pool_free(phip_ctx *ctx, void *ptr);
/* Same as phip_pool_free but addressed by context id; succeeds silently when
 * that context is already destroyed (its memory went with it).  This is the
 * deleter of a tensor handle that may outlive its device
 * (primitiv/core/memory_pool.h:22-35, test/cuda_device_test.cc:66-78). */
int phip_pool_free_by_id(uint64_t ctx_id, void *ptr);
int phip_pool_release_reserved(phip_ctx *ctx);
/* Bytes currently handed out / held in free lists, both pools of the context together. */
int phip_pool_stats(phip_ctx *ctx, uint64_t *supplied_bytes, uint64_t *reserved_bytes);

/* ---- copies ---------------------------------------------------------------
 * Reference: reset_tensor_by_array_impl (primitiv/devices/cuda/ops/
 * reset_tensor_by_array.cu:10-15), tensor_to_vector_impl (.../tensor_to_vector.cu:
 * 10-17), copy_tensor_impl (.../copy_tensor.cu:10-30).  h2d returns when the
 * host buffer may be reused; d2h returns when the data has arrived. */
int phip_memcpy_h2d(phip_ctx *ctx, void *dst, const void *src, size_t bytes);
int phip_memcpy_d2h(phip_ctx *ctx, void *dst, const void *src, size_t bytes);
int phip_memcpy_d2d(phip_ctx *ctx, void *dst, const void *src, size_t bytes);

/* ---- fill and storage conversion -----------------------------------------
 * Reference: reset_tensor_impl (primitiv/devices/cuda/ops/reset_tensor.cu:9-24,
 * primitiv/devices/cuda16/ops/reset_tensor.cu:9-24) and the fp32<->fp16 staging
 * kernels of the half-storage device (primitiv/devices/cuda16/ops/
 * reset_tensor_by_array.cu:9-30, .../tensor_to_vector.cu:9-32).
 * Conversions round to nearest even. */
int phip_fill_f32(phip_ctx *ctx, float *p, float value, size_t n);
int phip_fill_f16(phip_ctx *ctx, void *p, float value, size_t n);
int phip_fill_bf16(phip_ctx *ctx, void *p, float value, size_t n);
int phip_cvt_f32_to_f16(phip_ctx *ctx, const float *src, void *dst, size_t n);
int phip_cvt_f16_to_f32(phip_ctx *ctx, const void *src, float *dst, size_t n);
int phip_cvt_f32_to_bf16(phip_ctx *ctx, const float *src, void *dst, size_t n);
int phip_cvt_bf16_to_f32(phip_ctx *ctx, const void *src, float *dst, size_t n);

/* ---- y += x with minibatch broadcasting ------------------------------------
 * Reference: inplace_add_impl (primitiv/devices/eigen/ops/inplace_add.cc:9-23,
 * primitiv/devices/cuda/ops/inplace_add.cu:9-30, .../cuda16/ops/inplace_add.cu:
 * 9-40).  x holds `volume*bx` elements, y `volume*by`; bx == by, or one of
 * them is 1.  by == 1 < bx adds the sum of x over the minibatch. */
int phip_inplace_add_f32(phip_ctx *ctx, const float *x, float *y, uint32_t volume, uint32_t bx, uint32_t by);
int phip_inplace_add_f16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by);
int phip_inplace_add_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by);

/* ---- y[i] = sum over the minibatch of x[n][i] ------------------------------
 * Reference: batch_sum_fw_impl (primitiv/devices/eigen/ops/batch_sum.cc:9-22,
 * primitiv/devices/cuda/ops/batch_sum.cu:9-33, .../cuda16/ops/batch_sum.cu:9-33). */
int phip_batch_sum_f32(phip_ctx *ctx, const float *x, float *y, uint32_t volume, uint32_t bs);
int phip_batch_sum_f16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bs);
int phip_batch_sum_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bs);

/* ---- matmul forward:  y = a . b  per sample --------------------------------
 * Reference: Device::matmul_fw_impl (primitiv/core/device.h:464;
 * primitiv/devices/eigen/ops/matmul.cc:9-38; primitiv/devices/cuda/ops/matmul.cu:
 * 21-66; primitiv/devices/cuda16/ops/matmul.cu:46-126).
 * a: [di x dj] x ba, b: [dj x dk] x bb, y: [di x dk] x max(ba, bb); ba == bb
 * or one of them is 1.  y is overwritten and may be uninitialised on entry. */
int phip_matmul_fw_f32(phip_ctx *ctx, const float *a, const float *b, float *y,
                       uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);
int phip_matmul_fw_f16(phip_ctx *ctx, const void *a, const void *b, void *y,
                       uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);
int phip_matmul_fw_bf16(phip_ctx *ctx, const void *a, const void *b, void *y,
                        uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);

/* ---- matmul forward without any allocation ---------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device
 * memory during the call: tight serving loops, harnesses that forbid
 * hipMalloc, code that is being captured into a HIP graph.  (Capture has two
 * more conditions, which no test here exercises: the lanes switched off with
 * phip_set_overlap(ctx, 0), since an engaged lane records and waits for an
 * event, and one uncaptured call of the same shape beforehand, since the first
 * use of a kernel on a context sets a function attribute.)
 * Same arguments, kernels and result bits as
 * phip_matmul_fw_f32; a product whose K range is split between workgroups
 * keeps its partial tiles and tile counters in a fixed array inside the
 * library's device code (PHIP_NOALLOC_SCRATCH_BYTES per GPU, held until the
 * process ends) instead of a pool block.  Calls no hipMalloc / hipFree and
 * leaves the context's pool untouched.  A product that needs more scratch than
 * the array holds fails with PHIP_ERR_INVALID_ARGUMENT before anything has
 * been written to y.  All contexts on one GPU share that GPU's array: calls of
 * this entry point that overlap on one GPU (two contexts, i.e. two streams)
 * race; calls on one context are ordered by its stream. */
#define PHIP_NOALLOC_SCRATCH_BYTES (16u << 20)
int phip_matmul_fw_f32_noalloc(phip_ctx *ctx, const float *a, const float *b, float *y,
                               uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);

/* ---- matmul backward:  ga += gy . b^T ,  gb += a^T . gy --------------------
 * Reference: Device::matmul_bw_impl (primitiv/core/device.h:481-483;
 * primitiv/devices/eigen/ops/matmul.cc:40-79; primitiv/devices/cuda/ops/matmul.cu:
 * 68-139; primitiv/devices/cuda16/ops/matmul.cu:128-266).
 * Both gradients are accumulated into.  The gradient of an operand whose
 * batch is 1 is reduced over the minibatch inside the kernel (the reference's
 * CUDA device issues one GEMM per sample for that case, matmul.cu:113-123). */
int phip_matmul_bw_f32(phip_ctx *ctx, const float *a, const float *b, const float *gy,
                       float *ga, float *gb,
                       uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);
int phip_matmul_bw_f16(phip_ctx *ctx, const void *a, const void *b, const void *gy,
                       void *ga, void *gb,
                       uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);
int phip_matmul_bw_bf16(phip_ctx *ctx, const void *a, const void *b, const void *gy,
                        void *ga, void *gb,
                        uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb);

/* Which kernels the matrix products went to.  No counterpart in the reference
 * (its devices hand every product to a vendor GEMM).  Copies the names of the
 * GEMM kernels launched by this context's matmul and convolution calls since
 * the previous call into buf (space-separated, in launch order per stream;
 * truncated to buf_size; buf may be NULL), forgets them, and switches the
 * note-taking on (on != 0) or off (the default).  For benchmarks and tests
 * that report or assert the kernel family a shape is served by; costs nothing
 * while off. */
int phip_gemm_trace(phip_ctx *ctx, int on, char *buf, size_t buf_size);

/* ---- elementwise operations around the matmul ------------------------------
 * The layers of every primitiv example wrap the matmul in a bias add and an
 * activation (examples/mnist/mnist.cc:74,80; examples/ptb/ptb_rnnlm_lstm.cc:
 * 101-109), and the optimizers scale and subtract (primitiv/core/
 * optimizer_impl.cc:22-24).  These entry points stand behind the
 * corresponding Device virtuals (primitiv/core/device.h:393-479,531-534); an
 * operation code selects the member of a family.  Formulas follow
 * primitiv/devices/naive/ops/ and primitiv/devices/cuda/ops/ (file per code
 * named below).  All are streaming kernels: every operand an operation needs
 * is read once, every result written once; forward results overwrite,
 * gradients are accumulated into (`+=`), as in the reference.  The 16-bit
 * variants read and write 16-bit storage and compute in fp32
 * (primitiv/devices/cuda16/ops/common.h:16-113). */

/* y = f(x); gx += f'(x, y) * gy over n elements.
 * Reference: CUDADEV_KERNEL_FW_X / _BW_X (primitiv/devices/cuda/ops/common.h:
 * 14-28) instantiated in negate.cu, abs.cu, sqrt.cu, exp.cu, log.cu, tanh.cu,
 * sigmoid.cu, softplus.cu, sin.cu, cos.cu, tan.cu; same formulas in
 * primitiv/devices/naive/ops/.  The reference has no negate_bw, so
 * PHIP_NEGATE is forward only.  A backward call reads only those of x and y
 * that its formula uses; the other may be NULL. */
typedef enum phip_unary_op {
  PHIP_NEGATE = 0,
  PHIP_ABS = 1,
  PHIP_SQRT = 2,
  PHIP_EXP = 3,
  PHIP_LOG = 4,
  PHIP_TANH = 5,
  PHIP_SIGMOID = 6,
  PHIP_SOFTPLUS = 7,
  PHIP_SIN = 8,
  PHIP_COS = 9,
  PHIP_TAN = 10
} phip_unary_op;
int phip_unary_fw_f32(phip_ctx *ctx, int op, const float *x, float *y, size_t n);
int phip_unary_fw_f16(phip_ctx *ctx, int op, const void *x, void *y, size_t n);
int phip_unary_fw_bf16(phip_ctx *ctx, int op, const void *x, void *y, size_t n);
int phip_unary_bw_f32(phip_ctx *ctx, int op, const float *x, const float *y, const float *gy, float *gx, size_t n);
int phip_unary_bw_f16(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx, size_t n);
int phip_unary_bw_bf16(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx, size_t n);

/* y = f(x, k); gx += df/dx(x, y, k) * gy with a host constant k.
 * Reference: CUDADEV_KERNEL_FW_X_CONST / _BW_X_CONST (common.h:30-45) in
 * add.cu, subtract.cu, multiply.cu, divide.cu, pow.cu, prelu.cu, elu.cu.
 * _R: the constant is the right operand (x - k, x / k, x ^ k); _L: the left
 * (k - x, k / x, k ^ x).  PRELU: max(x,0) + k*min(x,0); ELU: max(x,0) +
 * k*(exp(min(x,0)) - 1). */
typedef enum phip_const_op {
  PHIP_ADD_CONST = 0,
  PHIP_SUBTRACT_CONST_R = 1,
  PHIP_SUBTRACT_CONST_L = 2,
  PHIP_MULTIPLY_CONST = 3,
  PHIP_DIVIDE_CONST_R = 4,
  PHIP_DIVIDE_CONST_L = 5,
  PHIP_POW_CONST_R = 6,
  PHIP_POW_CONST_L = 7,
  PHIP_PRELU = 8,
  PHIP_ELU = 9
} phip_const_op;
int phip_const_fw_f32(phip_ctx *ctx, int op, const float *x, float k, float *y, size_t n);
int phip_const_fw_f16(phip_ctx *ctx, int op, const void *x, float k, void *y, size_t n);
int phip_const_fw_bf16(phip_ctx *ctx, int op, const void *x, float k, void *y, size_t n);
int phip_const_bw_f32(phip_ctx *ctx, int op, const float *x, const float *y, const float *gy, float k, float *gx, size_t n);
int phip_const_bw_f16(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, float k, void *gx, size_t n);
int phip_const_bw_bf16(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, float k, void *gx, size_t n);

/* y = x ^ k for an integer k by repeated squaring; gx += k * gy * y / x.
 * Reference: pown_fw_impl / pown_bw_impl (primitiv/devices/cuda/ops/pown.cu:
 * 9-60, primitiv/devices/naive/ops/pown.cc:12-46). */
int phip_pown_fw_f32(phip_ctx *ctx, const float *x, int32_t k, float *y, size_t n);
int phip_pown_fw_f16(phip_ctx *ctx, const void *x, int32_t k, void *y, size_t n);
int phip_pown_fw_bf16(phip_ctx *ctx, const void *x, int32_t k, void *y, size_t n);
int phip_pown_bw_f32(phip_ctx *ctx, const float *x, const float *y, const float *gy, int32_t k, float *gx, size_t n);
int phip_pown_bw_f16(phip_ctx *ctx, const void *x, const void *y, const void *gy, int32_t k, void *gx, size_t n);
int phip_pown_bw_bf16(phip_ctx *ctx, const void *x, const void *y, const void *gy, int32_t k, void *gx, size_t n);

/* Binary operations with minibatch broadcasting.  a holds volume*ba elements,
 * b volume*bb, y volume*max(ba,bb); ba == bb or one of them is 1.
 * Forward: y = a op b.  Backward: ga += dy/da * gy, gb += dy/db * gy, where the
 * gradient of an operand whose batch is 1 is summed over the minibatch (the
 * reference does this with atomicAdd; here one workgroup owns each output
 * element and adds in a fixed order).  A backward call reads only those of
 * a, b, y that its formula uses; the others may be NULL.
 * Reference: CUDADEV_KERNEL_FW_AB (common.h:65-72) and the *_bw_dev kernels in
 * add.cu:16-27, subtract.cu, multiply.cu, divide.cu, pow.cu; primitiv/devices/naive/ops/{add,subtract,multiply,divide,
 * pow}.cc. */
typedef enum phip_binary_op {
  PHIP_ADD = 0,
  PHIP_SUBTRACT = 1,
  PHIP_MULTIPLY = 2,
  PHIP_DIVIDE = 3,
  PHIP_POW = 4
} phip_binary_op;
int phip_binary_fw_f32(phip_ctx *ctx, int op, const float *a, const float *b, float *y, uint32_t volume, uint32_t ba, uint32_t bb);
int phip_binary_fw_f16(phip_ctx *ctx, int op, const void *a, const void *b, void *y, uint32_t volume, uint32_t ba, uint32_t bb);
int phip_binary_fw_bf16(phip_ctx *ctx, int op, const void *a, const void *b, void *y, uint32_t volume, uint32_t ba, uint32_t bb);
int phip_binary_bw_f32(phip_ctx *ctx, int op, const float *a, const float *b, const float *y, const float *gy,
                       float *ga, float *gb, uint32_t volume, uint32_t ba, uint32_t bb);
int phip_binary_bw_f16(phip_ctx *ctx, int op, const void *a, const void *b, const void *y, const void *gy,
                       void *ga, void *gb, uint32_t volume, uint32_t ba, uint32_t bb);
int phip_binary_bw_bf16(phip_ctx *ctx, int op, const void *a, const void *b, const void *y, const void *gy,
                       void *ga, void *gb, uint32_t volume, uint32_t ba, uint32_t bb);

/* y = x op k (k_on_left == 0) or k op x (k_on_left != 0), where k holds one
 * scalar per sample: x has volume*bx elements, k has bk, y volume*max(bx,bk).
 * Reference: CUDADEV_KERNEL_FW_X_SCALAR_R / _L (common.h:47-63) for
 * add_scalar, subtract_scalar_{r,l}, multiply_scalar, divide_scalar_{r,l},
 * pow_scalar_{r,l}; CPUDEV_FW_X_SCALAR (primitiv/devices/naive/ops/common.h:
 * 50-68). */
int phip_scalar_fw_f32(phip_ctx *ctx, int op, int k_on_left, const float *x, const float *k, float *y,
                       uint32_t volume, uint32_t bx, uint32_t bk);
int phip_scalar_fw_f16(phip_ctx *ctx, int op, int k_on_left, const void *x, const void *k, void *y,
                       uint32_t volume, uint32_t bx, uint32_t bk);
int phip_scalar_fw_bf16(phip_ctx *ctx, int op, int k_on_left, const void *x, const void *k, void *y,
                       uint32_t volume, uint32_t bx, uint32_t bk);

/* y -= x with minibatch broadcasting (same operand rules as phip_inplace_add).
 * Reference: inplace_subtract_impl (primitiv/devices/cuda/ops/
 * inplace_subtract.cu:9-27, primitiv/devices/naive/ops/inplace_subtract.cc:
 * 11-27). */
int phip_inplace_subtract_f32(phip_ctx *ctx, const float *x, float *y, uint32_t volume, uint32_t bx, uint32_t by);
int phip_inplace_subtract_f16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by);
int phip_inplace_subtract_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by);

/* x *= k over n elements.
 * Reference: inplace_multiply_const_impl (primitiv/devices/cuda/ops/
 * inplace_multiply_const.cu:9-23). */
int phip_inplace_multiply_const_f32(phip_ctx *ctx, float k, float *x, size_t n);
int phip_inplace_multiply_const_f16(phip_ctx *ctx, float k, void *x, size_t n);
int phip_inplace_multiply_const_bf16(phip_ctx *ctx, float k, void *x, size_t n);

/* y = identity matrix of `rows` x `rows`.
 * Reference: identity_impl (primitiv/devices/cuda/ops/identity.cu:9-22). */
int phip_identity_f32(phip_ctx *ctx, float *y, uint32_t rows);
int phip_identity_f16(phip_ctx *ctx, void *y, uint32_t rows);
int phip_identity_bf16(phip_ctx *ctx, void *y, uint32_t rows);

/* ---- moving and reducing along one dimension ---------------------------------
 * The operations the recurrent and language-model graphs of the reference put
 * between their matmuls (examples/ptb/ptb_rnnlm_lstm.cc:101-103,146-154;
 * softmax cross entropy is logsumexp + broadcast + pick, primitiv/core/
 * tensor_funcs.cc:310-329).  Around a dimension `dim` a tensor is seen as
 * [outer][n][base]: base = product of the dimensions below dim
 * (Shape::lower_volume), n = its extent along dim, outer = everything above,
 * the minibatch included; element (o, j, i) lives at (o*n + j)*base + i. */

/* dst[b][r][i] (= or +=) src[b][r][i] for i < span, r < rows, b < bs, with
 * element offsets b*bstride + r*stride + i on either side.  A batch stride of
 * 0 broadcasts the source, or - accumulating only - sums every sample into
 * the one destination (added in order of b by the thread that owns the
 * element).  Stands behind slice_fw/bw, concat_fw, batch_slice_fw/bw and
 * batch_concat_fw, which differ only in the offsets their host side passes
 * (primitiv/devices/cuda/ops/slice.cu:9-57, concat.cu:9-42, batch_slice.cu:
 * 9-47, batch_concat.cu:9-32; primitiv/devices/naive/ops/slice.cc:11-56,
 * concat.cc:11-37). */
int phip_copy_rows_f32(phip_ctx *ctx, const float *src, float *dst, uint32_t span, uint32_t rows,
                       uint64_t src_stride, uint64_t dst_stride, uint32_t bs,
                       uint64_t src_bstride, uint64_t dst_bstride, int accumulate);
int phip_copy_rows_f16(phip_ctx *ctx, const void *src, void *dst, uint32_t span, uint32_t rows,
                       uint64_t src_stride, uint64_t dst_stride, uint32_t bs,
                       uint64_t src_bstride, uint64_t dst_bstride, int accumulate);
int phip_copy_rows_bf16(phip_ctx *ctx, const void *src, void *dst, uint32_t span, uint32_t rows,
                       uint64_t src_stride, uint64_t dst_stride, uint32_t bs,
                       uint64_t src_bstride, uint64_t dst_bstride, int accumulate);

/* pick: y[b][o][0][i] = x[b or 0][o][ids[b or 0]][i]; x is [outer][n][base]
 * per sample with bx samples, y has bs = max(bx, n_ids) samples; `ids` is a
 * HOST array of n_ids indices (n_ids == bs, or 1 to use the same index for
 * every sample), each < n.  Backward: gx[...] += gy, summed over the samples
 * when bx == 1 (in order of b, no atomics).
 * Reference: pick_fw_impl / pick_bw_impl (primitiv/devices/cuda/ops/pick.cu:
 * 9-72, primitiv/devices/naive/ops/pick.cc:11-52). */
int phip_pick_fw_f32(phip_ctx *ctx, const float *x, const uint32_t *ids, uint32_t n_ids, float *y,
                     uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs);
int phip_pick_fw_f16(phip_ctx *ctx, const void *x, const uint32_t *ids, uint32_t n_ids, void *y,
                     uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs);
int phip_pick_fw_bf16(phip_ctx *ctx, const void *x, const uint32_t *ids, uint32_t n_ids, void *y,
                     uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs);
int phip_pick_bw_f32(phip_ctx *ctx, const float *gy, const uint32_t *ids, uint32_t n_ids, float *gx,
                     uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs);
int phip_pick_bw_f16(phip_ctx *ctx, const void *gy, const uint32_t *ids, uint32_t n_ids, void *gx,
                     uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs);
int phip_pick_bw_bf16(phip_ctx *ctx, const void *gy, const uint32_t *ids, uint32_t n_ids, void *gx,
                     uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs);

/* batch_pick: y[b] = x[ids[b]] for whole samples of `volume` elements (x has
 * bx samples, ids is a HOST array of n_ids indices < bx); backward
 * gx[ids[b]] += gy[b] in order of b.
 * Reference: batch_pick_fw_impl / batch_pick_bw_impl (primitiv/devices/cuda/
 * ops/batch_pick.cu:9-58, primitiv/devices/naive/ops/batch_pick.cc:11-34). */
int phip_batch_pick_fw_f32(phip_ctx *ctx, const float *x, const uint32_t *ids, uint32_t n_ids, float *y,
                           uint32_t volume, uint32_t bx);
int phip_batch_pick_fw_f16(phip_ctx *ctx, const void *x, const uint32_t *ids, uint32_t n_ids, void *y,
                           uint32_t volume, uint32_t bx);
int phip_batch_pick_fw_bf16(phip_ctx *ctx, const void *x, const uint32_t *ids, uint32_t n_ids, void *y,
                           uint32_t volume, uint32_t bx);
int phip_batch_pick_bw_f32(phip_ctx *ctx, const float *gy, const uint32_t *ids, uint32_t n_ids, float *gx,
                           uint32_t volume, uint32_t bx);
int phip_batch_pick_bw_f16(phip_ctx *ctx, const void *gy, const uint32_t *ids, uint32_t n_ids, void *gx,
                           uint32_t volume, uint32_t bx);
int phip_batch_pick_bw_bf16(phip_ctx *ctx, const void *gy, const uint32_t *ids, uint32_t n_ids, void *gx,
                           uint32_t volume, uint32_t bx);

/* Matrix transpose per sample: x is rows x cols, y cols x rows (column-major);
 * backward gx += transpose(gy) with gx rows x cols.
 * Reference: transpose_fw_impl / transpose_bw_impl (primitiv/devices/cuda/ops/
 * transpose.cu:9-54). */
int phip_transpose_fw_f32(phip_ctx *ctx, const float *x, float *y, uint32_t rows, uint32_t cols, uint32_t bs);
int phip_transpose_fw_f16(phip_ctx *ctx, const void *x, void *y, uint32_t rows, uint32_t cols, uint32_t bs);
int phip_transpose_fw_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t rows, uint32_t cols, uint32_t bs);
int phip_transpose_bw_f32(phip_ctx *ctx, const float *gy, float *gx, uint32_t rows, uint32_t cols, uint32_t bs);
int phip_transpose_bw_f16(phip_ctx *ctx, const void *gy, void *gx, uint32_t rows, uint32_t cols, uint32_t bs);
int phip_transpose_bw_bf16(phip_ctx *ctx, const void *gy, void *gx, uint32_t rows, uint32_t cols, uint32_t bs);

/* permute_dims: y's dimension i is x's dimension perm[i]; `dims` are x's
 * ndims <= 8 extents, `perm` a permutation of 0..ndims-1 (HOST arrays).
 * Backward: gx += the inverse permutation of gy.
 * Reference: permute_dims_fw_impl / _bw_impl (primitiv/devices/cuda/ops/
 * permute_dims.cu:9-115, primitiv/devices/naive/ops/permute_dims.cc:11-84). */
int phip_permute_dims_fw_f32(phip_ctx *ctx, const float *x, float *y, uint32_t ndims, const uint32_t *dims,
                             const uint32_t *perm, uint32_t bs);
int phip_permute_dims_fw_f16(phip_ctx *ctx, const void *x, void *y, uint32_t ndims, const uint32_t *dims,
                             const uint32_t *perm, uint32_t bs);
int phip_permute_dims_fw_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t ndims, const uint32_t *dims,
                             const uint32_t *perm, uint32_t bs);
int phip_permute_dims_bw_f32(phip_ctx *ctx, const float *gy, float *gx, uint32_t ndims, const uint32_t *dims,
                             const uint32_t *perm, uint32_t bs);
int phip_permute_dims_bw_f16(phip_ctx *ctx, const void *gy, void *gx, uint32_t ndims, const uint32_t *dims,
                             const uint32_t *perm, uint32_t bs);
int phip_permute_dims_bw_bf16(phip_ctx *ctx, const void *gy, void *gx, uint32_t ndims, const uint32_t *dims,
                             const uint32_t *perm, uint32_t bs);

/* flip: y[o][j][i] = x[o][n-1-j][i]; backward gx[o][j][i] += gy[o][n-1-j][i].
 * Reference: flip_fw_impl / flip_bw_impl (primitiv/devices/cuda/ops/flip.cu:
 * 9-63). */
int phip_flip_fw_f32(phip_ctx *ctx, const float *x, float *y, uint32_t base, uint32_t n, uint32_t outer);
int phip_flip_fw_f16(phip_ctx *ctx, const void *x, void *y, uint32_t base, uint32_t n, uint32_t outer);
int phip_flip_fw_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t base, uint32_t n, uint32_t outer);
int phip_flip_bw_f32(phip_ctx *ctx, const float *gy, float *gx, uint32_t base, uint32_t n, uint32_t outer);
int phip_flip_bw_f16(phip_ctx *ctx, const void *gy, void *gx, uint32_t base, uint32_t n, uint32_t outer);
int phip_flip_bw_bf16(phip_ctx *ctx, const void *gy, void *gx, uint32_t base, uint32_t n, uint32_t outer);

/* broadcast: y[o][j][i] = x[o][i] for j < size.
 * Reference: broadcast_fw_impl (primitiv/devices/cuda/ops/broadcast.cu:9-33). */
int phip_broadcast_fw_f32(phip_ctx *ctx, const float *x, float *y, uint32_t base, uint32_t size, uint32_t outer);
int phip_broadcast_fw_f16(phip_ctx *ctx, const void *x, void *y, uint32_t base, uint32_t size, uint32_t outer);
int phip_broadcast_fw_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t base, uint32_t size, uint32_t outer);

/* Reductions along dim: y[o][i] = op over j < n of x[o][j][i].  The partial
 * results of the threads that share an output are combined in a fixed order.
 * Reference: sum_fw_impl, logsumexp_fw_impl, max_fw_impl, min_fw_impl
 * (primitiv/devices/cuda/ops/sum.cu:9-70, logsumexp.cu:9-80, max.cu:9-43,
 * 99-123, min.cu; primitiv/devices/naive/ops/{sum,logsumexp,max,min}.cc). */
typedef enum phip_reduce_op {
  PHIP_SUM = 0,
  PHIP_LOGSUMEXP = 1,
  PHIP_MAX = 2,
  PHIP_MIN = 3
} phip_reduce_op;
int phip_reduce_fw_f32(phip_ctx *ctx, int op, const float *x, float *y, uint32_t base, uint32_t n, uint32_t outer);
int phip_reduce_fw_f16(phip_ctx *ctx, int op, const void *x, void *y, uint32_t base, uint32_t n, uint32_t outer);
int phip_reduce_fw_bf16(phip_ctx *ctx, int op, const void *x, void *y, uint32_t base, uint32_t n, uint32_t outer);

/* max_bw / min_bw (op = PHIP_MAX or PHIP_MIN): gx[o][j*][i] += gy[o][i], j*
 * the first j with x[o][j][i] == y[o][i].
 * Reference: max_bw_impl / min_bw_impl (primitiv/devices/cuda/ops/max.cu:
 * 45-97,125-151, primitiv/devices/naive/ops/max.cc:33-55). */
int phip_extremum_bw_f32(phip_ctx *ctx, int op, const float *x, const float *y, const float *gy, float *gx,
                         uint32_t base, uint32_t n, uint32_t outer);
int phip_extremum_bw_f16(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx,
                         uint32_t base, uint32_t n, uint32_t outer);
int phip_extremum_bw_bf16(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx,
                         uint32_t base, uint32_t n, uint32_t outer);

/* argmax / argmin (op = PHIP_MAX or PHIP_MIN): host_out[o*base + i] = the
 * first j attaining the extremum; blocks until the indices are on the host.
 * Reference: argmax_impl / argmin_impl (primitiv/devices/cuda/ops/argmax.cu:
 * 9-98, primitiv/devices/naive/ops/argmax.cc:11-36). */
int phip_arg_extremum_f32(phip_ctx *ctx, int op, const float *x, uint32_t *host_out,
                          uint32_t base, uint32_t n, uint32_t outer);
int phip_arg_extremum_f16(phip_ctx *ctx, int op, const void *x, uint32_t *host_out,
                          uint32_t base, uint32_t n, uint32_t outer);
int phip_arg_extremum_bf16(phip_ctx *ctx, int op, const void *x, uint32_t *host_out,
                          uint32_t base, uint32_t n, uint32_t outer);

/* ---- random tensors ----------------------------------------------------------
 * Reference: random_bernoulli_impl, random_uniform_impl, random_normal_impl,
 * random_log_normal_impl (primitiv/core/device.h:381-384; primitiv/devices/
 * cuda/ops/random_{bernoulli,uniform,normal,log_normal}.cu): uniform draws in
 * (lower, upper], Bernoulli as (u <= p) with u in (0, 1], normal and
 * log-normal with (mean, sd).  The reference's GPU device takes its stream
 * from cuRAND; here the stream is Philox4x32-10 (Salmon et al., SC'11),
 * stateless: element i is word i%4 of the block with counter offset + i/4
 * under the key `seed`.  The caller owns the position in the stream and moves
 * `offset` on by (n + 3) / 4 after a call; a call with a smaller n yields a
 * prefix of the same draw.  Normal draws use Box-Muller on word pairs. */
int phip_random_uniform_f32(phip_ctx *ctx, uint64_t seed, uint64_t offset, float lower, float upper,
                            float *y, size_t n);
int phip_random_uniform_f16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float lower, float upper,
                            void *y, size_t n);
int phip_random_uniform_bf16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float lower, float upper,
                            void *y, size_t n);
int phip_random_bernoulli_f32(phip_ctx *ctx, uint64_t seed, uint64_t offset, float p, float *y, size_t n);
int phip_random_bernoulli_f16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float p, void *y, size_t n);
int phip_random_bernoulli_bf16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float p, void *y, size_t n);
int phip_random_normal_f32(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd,
                           float *y, size_t n);
int phip_random_normal_f16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd,
                           void *y, size_t n);
int phip_random_normal_bf16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd,
                           void *y, size_t n);
int phip_random_log_normal_f32(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd,
                               float *y, size_t n);
int phip_random_log_normal_f16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd,
                               void *y, size_t n);
int phip_random_log_normal_bf16(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd,
                               void *y, size_t n);

/* ---- convolution and pooling -----------------------------------------------
 * conv2d: x is x0 x x1 x c per sample (first dimension contiguous), w is
 * w0 x w1 x c x oc, y is y0 x y1 x oc with y0 = (x0 + 2 pad0 - ((w0-1) dil0 + 1))
 * / str0 + 1 and y1 likewise (primitiv/core/shape_ops.cc:162-187); bx and bw
 * are the minibatch sizes of x and w (equal, or 1 = shared by all samples).
 * A true convolution: the tap at window offset (i, j) meets kernel element
 * (w0-1-i, w1-1-j).  Forward overwrites y; backward adds to gx (shape of x) and
 * gw (shape of w), a shared operand's gradient collecting every sample.
 * Scratch comes from the context's pool.
 * Reference: conv2d_fw_impl / conv2d_bw_impl (primitiv/devices/naive/ops/
 * conv2d.cc:9-151 for the arithmetic, primitiv/devices/cuda/ops/conv2d.cu:11-198
 * for the device interface). */
int phip_conv2d_fw_f32(phip_ctx *ctx, const float *x, const float *w, float *y, uint32_t x0, uint32_t x1,
    uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1,
    uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);
int phip_conv2d_bw_f32(phip_ctx *ctx, const float *x, const float *w, const float *gy, float *gx, float *gw,
    uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw,
    uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);
int phip_conv2d_fw_f16(phip_ctx *ctx, const void *x, const void *w, void *y, uint32_t x0, uint32_t x1,
    uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1,
    uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);
int phip_conv2d_bw_f16(phip_ctx *ctx, const void *x, const void *w, const void *gy, void *gx, void *gw,
    uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw,
    uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);
int phip_conv2d_fw_bf16(phip_ctx *ctx, const void *x, const void *w, void *y, uint32_t x0, uint32_t x1,
    uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1,
    uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);
int phip_conv2d_bw_bf16(phip_ctx *ctx, const void *x, const void *w, const void *gy, void *gx, void *gw,
    uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw,
    uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);

/* max_pool2d over `repeat` planes of x0 x x1 (channels times minibatch): y is
 * y0 x y1 per plane with y0 = (x0 + 2 pad0 - win0) / str0 + 1 and y1 likewise
 * (shape_ops.cc:189-213); padding never wins.  Backward adds gy to the FIRST
 * element of each window (second window axis outer, first inner) that equals
 * y; the same bits on every run.
 * Reference: max_pool2d_fw_impl / max_pool2d_bw_impl (primitiv/devices/naive/ops/
 * max_pool2d.cc:9-113, primitiv/devices/cuda/ops/max_pool2d.cu:11-117). */
int phip_max_pool2d_fw_f32(phip_ctx *ctx, const float *x, float *y, uint32_t x0, uint32_t x1, uint32_t repeat,
    uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1);
int phip_max_pool2d_bw_f32(phip_ctx *ctx, const float *x, const float *y, const float *gy, float *gx,
    uint32_t x0, uint32_t x1, uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1,
    uint32_t str0, uint32_t str1);
int phip_max_pool2d_fw_f16(phip_ctx *ctx, const void *x, void *y, uint32_t x0, uint32_t x1, uint32_t repeat,
    uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1);
int phip_max_pool2d_bw_f16(phip_ctx *ctx, const void *x, const void *y, const void *gy, void *gx, uint32_t x0,
    uint32_t x1, uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0,
    uint32_t str1);
int phip_max_pool2d_fw_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t x0, uint32_t x1, uint32_t repeat,
    uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1);
int phip_max_pool2d_bw_bf16(phip_ctx *ctx, const void *x, const void *y, const void *gy, void *gx, uint32_t x0,
    uint32_t x1, uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0,
    uint32_t str1);

/* ---- timing ---------------------------------------------------------------
 * No counterpart in the reference (it has no profiling facility); events are
 * recorded on the context's stream so they bracket exactly the kernels the
 * library launched. */
int phip_event_create(phip_ctx *ctx, phip_event **out);
int phip_event_destroy(phip_event *ev);
int phip_event_record(phip_ctx *ctx, phip_event *ev);
/* Waits for `stop`, then returns the milliseconds between the two events. */
int phip_event_elapsed_ms(phip_event *start, phip_event *stop, float *ms);

/* ---- host-side seeded inputs ----------------------------------------------
 * Reference: DefaultRandomizer (primitiv/core/random.h:15-87), the generator
 * behind the CPU devices' random_* ops: std::mt19937 with one freshly built
 * standard-library distribution per fill.  uniform yields (lower, upper].
 * These run on the host and write host memory; they exist so that every
 * device is handed bit-identical seeded inputs. */
int phip_randomizer_create(uint32_t seed, phip_randomizer **out);
int phip_randomizer_destroy(phip_randomizer *r);
int phip_randomizer_fill_uniform(phip_randomizer *r, float lower, float upper, size_t n, float *host_out);
int phip_randomizer_fill_normal(phip_randomizer *r, float mean, float sd, size_t n, float *host_out);

#ifdef __cplusplus
}
#endif

#endif /* PHIP_H_ */
