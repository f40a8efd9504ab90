/*
 * bship.h - C ABI of libbship.so, the MI355X (gfx950) compute back end behind
 * brainstorm's Handler interface.
 *
 * Every entry point is what a ctypes/cffi binding of the reference's handler
 * would bind for one handler operation; the comment above each declaration
 * names the reference method it stands in for
 * (brainstorm/handlers/numpy_handler.py = "numpy", pycuda_handler.py = "pycuda",
 * base_handler.py = "base", _cpuop.pyx = "_cpuop").
 *
 * Conventions
 *  - extern "C", C99 types only, no exceptions cross the boundary.
 *  - Every function returns an int status: 0 = OK, > 0 = a hipError_t,
 *    < 0 = one of the BSHIP_ERR_* argument/state errors below. The message of
 *    the last failure on the calling thread is returned by bship_last_error().
 *  - Pointers named float* / void* are raw DEVICE addresses (already offset to
 *    the first element of the view) unless the parameter is called `host`.
 *    All arrays are dense, C-contiguous float32. Only 4-byte alignment is
 *    required; 16-byte aligned pointers take the fastest kernels.
 *  - An output may be the same array as an input for every elementwise and
 *    broadcast operation (in-place use); partial overlap is not supported.
 *  - All work is enqueued, in call order, on one stream owned by the library.
 *    Calls return without waiting unless stated ("blocks").
 *  - Zero-sized arrays (n == 0, M == 0 ...) are legal and do nothing.
 */
#ifndef BSHIP_H
#define BSHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BSHIP_VERSION 300 /* major*10000 + minor*100 + patch */

/* argument / state errors (negative so they never collide with hipError_t) */
#define BSHIP_ERR_NOT_INITIALIZED (-1)
#define BSHIP_ERR_NULL_POINTER    (-2)
#define BSHIP_ERR_BAD_DIMENSION   (-3)
#define BSHIP_ERR_BAD_OP          (-4)
#define BSHIP_ERR_OUT_OF_MEMORY   (-5)
#define BSHIP_ERR_UNSUPPORTED     (-6)
#define BSHIP_ERR_BAD_POINTER     (-7)
#define BSHIP_ERR_BLAS            (-8)
#define BSHIP_ERR_TIMEOUT         (-9)   /* a bounded wait inside a kernel ran out; every kernel has exited */

/* ------------------------------ lifecycle -------------------------------- */

/* Selects the device, creates the stream and the memory pool. Idempotent for
 * the same device. Replaces `import pycuda.autoinit` + culinalg.init()
 * (pycuda 18; brainstorm/optional.py 32). */
int bship_init(int device);
/* Frees every pool block and destroys the stream. Blocks. */
int bship_shutdown(void);
/* Waits for all enqueued work. Blocks. */
int bship_sync(void);
int bship_version(void);
/* Message of the last failed call on this thread ("" if none). The string is
 * owned by the library and valid until the next failing call on the thread. */
const char* bship_last_error(void);
/* Device name and compute-unit count of the initialised device. */
int bship_device_info(char* name_host, size_t name_len, int* compute_units);

/* Timing on the library's stream, where the kernels actually run: record
 * enqueues a hipEvent into one of BSHIP_MAX_EVENTS slots (no waiting);
 * elapsed waits for slot `stop` and returns the time between the two records. */
#define BSHIP_MAX_EVENTS 1024
int bship_event_record(int slot);
int bship_event_elapsed_ms(int start_slot, int stop_slot, float* ms_host);

/* Recorded steps. The reference's trainer issues every handler call of a
 * training step one by one from Python (trainer.py 83-100, steppers.py 60-140,
 * network.py 409-460); small networks are bound by that, not by the device.
 * Between bship_graph_begin and bship_graph_end the calls of this library are
 * recorded (HIP stream capture) instead of executed; bship_graph_launch then
 * replays the whole recording with one launch, on the library's stream and in
 * order with every other call. A recording may contain compute calls, device
 * to device copies, bship_malloc and bship_free (blocks handed out while
 * recording stay reserved for the graph until it is destroyed). Calls that wait
 * for the device or touch host memory (bship_sync, bship_h2d, bship_d2h, timers,
 * bship_isfinite_f32, bship_fill_gaussian_f32, bship_rng_seed,
 * bship_rng_get_state, bship_pool_trim) return BSHIP_ERR_UNSUPPORTED while
 * recording. Dropout masks of a recorded step continue the random stream
 * exactly as eager calls would (replay r uses the draws that follow those of
 * replay r-1; other uses of the generator between replays are allowed). */
int bship_graph_begin(void);
int bship_graph_end(int* graph_id);
int bship_graph_launch(int graph_id);
int bship_graph_destroy(int graph_id);

/* ------------------------------- memory ---------------------------------- */

/* allocate/zeros (numpy 36-43, pycuda 70-79): a block of at least `nbytes`
 * from the caching pool, 256-byte aligned and ZERO-FILLED (both reference
 * handlers return zeros from allocate, and lstm_layer.py 167/258 depends on
 * it). nbytes == 0 yields *out = NULL and status 0. */
int bship_malloc(size_t nbytes, void** out);
/* The same without the zero fill, for buffers that their owner overwrites
 * completely before reading them (the col matrix of conv2d_*_batch, numpy 122
 * and 156-157, which the reference allocates once per image; upload targets).
 * The content is whatever the block's previous owner left. */
int bship_malloc_scratch(size_t nbytes, void** out);
/* Returns a block to the pool cache (no hipFree). NULL is a no-op. */
int bship_free(void* p);
/* hipFree()s every cached (unused) block. Blocks. */
int bship_pool_trim(void);
int bship_pool_stats(size_t* bytes_in_use, size_t* bytes_cached,
                     size_t* device_allocations);

/* set_from_numpy / create_from_numpy (numpy 54-65, pycuda 90-107). Blocks
 * until the host buffer may be reused. */
int bship_h2d(void* dst, const void* src_host, size_t nbytes);
/* get_numpy_copy (numpy 60-62, pycuda 99-101). Blocks. */
int bship_d2h(void* dst_host, const void* src, size_t nbytes);
/* copy_to (numpy 47-52, pycuda 83-85). */
int bship_d2d(void* dst, const void* src, size_t nbytes);
/* Copy between row-pitched matrices: dst(rows, cols) with ld_dst elements from one
 * row to the next = src(rows, cols) with ld_src. This is how a feature slice of a
 * hub that several layers write side by side (buffer_structure.py 232-245), which
 * NumPy addresses with strides, is moved into and out of the dense form that the
 * kernels work on. */
int bship_copy2d_f32(float* dst, int64_t ld_dst, const float* src, int64_t ld_src,
                     int64_t rows, int64_t cols);
/* fill (numpy 57-58, pycuda 93-94). */
int bship_fill_f32(float* mem, float val, size_t n);

/* ----------------------------- elementwise ------------------------------- */

enum {
    BSHIP_ADD = 0,  /* add_tt       numpy 86-87   pycuda 130-131 */
    BSHIP_SUB = 1,  /* subtract_tt  numpy 264-266 pycuda 372-373 */
    BSHIP_MUL = 2,  /* mult_tt      numpy 245-246 pycuda 351-352 */
    BSHIP_DIV = 3,  /* divide_tt    numpy 190-191 pycuda 272-273 */
    BSHIP_FMOD = 4  /* modulo_tt    numpy 227-228 (np.fmod: sign of dividend) */
};
/* out = a (op) b */
int bship_binary_f32(int op, const float* a, const float* b, float* out, size_t n);

/* mult_add_tt (numpy 233-234, pycuda 331-332): out += a*b, the product rounded
 * to float32 before the add exactly as NumPy evaluates it (no fused multiply-add). */
int bship_mult_add_tt_f32(const float* a, const float* b, float* out, size_t n);

enum {
    BSHIP_ADD_ST = 0,      /* add_st       numpy 83-84   : out = t + s   */
    BSHIP_MULT_ST = 1,     /* mult_st      numpy 242-243 : out = s * t   */
    BSHIP_MULT_ADD_ST = 2  /* mult_add_st  numpy 230-231 : out += s * t  */
};
/* The Python float scalar is rounded to float32 first, which is what NumPy
 * does for a float32 array combined with a Python scalar. */
int bship_scalar_f32(int op, float s, const float* t, float* out, size_t n);

enum {
    BSHIP_ABS = 0,     /* abs_t   numpy 74-75   */
    BSHIP_SIGN = 1,    /* sign_t  numpy 248-249 */
    BSHIP_SQRT = 2,    /* sqrt_t  numpy 258-259 */
    BSHIP_LOG = 3,     /* log_t   numpy 207-208 */
    BSHIP_SIGMOID = 4, /* sigmoid numpy 283-287 */
    BSHIP_TANH = 5,    /* tanh    numpy 297-298 */
    BSHIP_REL = 6,     /* rel     numpy 277-278 : x*(x>0), negatives give -0.0 */
    BSHIP_EL = 7       /* el      numpy 303-305 */
};
int bship_unary_f32(int op, const float* x, float* y, size_t n);

enum {
    BSHIP_SIGMOID_DERIV = 0, /* numpy 289-290 : dx = (dy*y)*(1-y)          */
    BSHIP_TANH_DERIV = 1,    /* numpy 300-301 : dx = dy*(1-y*y)            */
    BSHIP_REL_DERIV = 2,     /* numpy 280-281 : dx = dy*(y>0)              */
    BSHIP_EL_DERIV = 3       /* numpy 307-309 : dx = dy*(y>=0)+dy*(y+1)*(y<0) */
};
/* The reference never reads `x` in a derivative, so it is not passed. */
int bship_deriv_f32(int op, const float* y, const float* dy, float* dx, size_t n);

/* clip_t (numpy 107-108, pycuda 171-172) */
int bship_clip_f32(const float* a, float lo, float hi, float* out, size_t n);

enum {
    BSHIP_COPY_IF = 0, /* copy_to_if  numpy 173-174 : if cond!=0: out = a    */
    BSHIP_FILL_IF = 1, /* fill_if     numpy 196-197 : if cond!=0: out = val  */
    BSHIP_ADD_IF = 2   /* add_into_if numpy 77-78   : if cond!=0: out += a   */
};
/* `a` is ignored for FILL_IF, `val` for the other two. */
int bship_cond_f32(int op, const float* a, float val, float* out,
                   const float* cond, size_t n);

/* ------------------------------ broadcast -------------------------------- */

/* add_mv / subtract_mv / mult_mv / divide_mv (numpy 80-81, 261-262, 236-237,
 * 187-188; pycuda 124-125, 369-370, 334-338, 269-270) and mult_add_mv
 * (numpy 239-240): m is (M,N); v is (1,N) when v_is_col == 0, (M,1) otherwise.
 * op is BSHIP_ADD/SUB/MUL/DIV. accumulate != 0 computes out += m (op) v. */
int bship_mv_f32(int op, const float* m, const float* v, float* out,
                 int64_t M, int64_t N, int v_is_col, int accumulate);

/* broadcast_t (numpy 103-105, pycuda 166-169): a has shape (outer,1,inner),
 * out has shape (outer,bdim,inner). */
int bship_broadcast_f32(const float* a, float* out, int64_t outer,
                        int64_t bdim, int64_t inner);

/* broadcast_t between arrays made of contiguous runs (feature slices of wider hubs):
 * dense element k of an array lies at (k / run) * ld + k % run. outer * inner must be a
 * whole number of runs of a, the whole output a whole number of runs of out. At most
 * 2^32 - 1 output elements. */
int bship_broadcast_pitched_f32(const float* a, int64_t a_run, int64_t ld_a, float* out,
                                int64_t out_run, int64_t ld_out, int64_t outer, int64_t bdim,
                                int64_t inner);
/* merge_tt (numpy 221-225, pycuda 317-323): out[:, :na] = a, out[:, na:] = b */
int bship_merge_f32(const float* a, const float* b, float* out, int64_t rows,
                    int64_t na, int64_t nb);
/* split_add_tt (numpy 251-256, pycuda 357-364): oa += x[:, :na]; ob += x[:, na:] */
int bship_split_add_f32(const float* x, float* oa, float* ob, int64_t rows,
                        int64_t na, int64_t nb);

/* ------------------------- row-pitched operands -------------------------- */

/* Every elementwise operation above, and the matrix (op) vector operations, on
 * (rows, cols) operands whose rows lie a pitch apart: the feature slices
 * hub[:, :, a:b] of a hub that several layers write side by side
 * (buffer_structure.py 232-245), which NumpyHandler reaches through NumPy's
 * strides (numpy_handler.py: the same lines as the dense forms).
 * `family` selects the dense entry point whose arithmetic is applied and `op`
 * its operation code; the results equal the dense ones bit for bit.
 *   family                 op codes of            inputs                 scalars
 *   BSHIP_PITCHED_BINARY   bship_binary_f32       a, b                   -
 *   BSHIP_PITCHED_MULT_ADD -                      a, b   (out += a*b)    -
 *   BSHIP_PITCHED_SCALAR   bship_scalar_f32       a = t                  s0 = s
 *   BSHIP_PITCHED_UNARY    bship_unary_f32        a = x                  -
 *   BSHIP_PITCHED_DERIV    bship_deriv_f32        a = y, b = dy          -
 *   BSHIP_PITCHED_CLIP     -                      a                      s0 = lo, s1 = hi
 *   BSHIP_PITCHED_COND     bship_cond_f32         a (not FILL_IF), b = cond   s0 = val
 *   BSHIP_PITCHED_FILL     -                      -                      s0 = val
 * An input is a matrix (row stride = its pitch in elements, column stride 1),
 * a row vector (row stride 0, column stride 1) or a column vector (row stride
 * 1, column stride 0): with a vector for b, BINARY is add_mv / subtract_mv /
 * mult_mv / divide_mv and MULT_ADD is mult_add_mv. out is (rows, cols) with
 * ld_out elements from one row to the next and may be one of the inputs. */
enum {
    BSHIP_PITCHED_BINARY = 0,
    BSHIP_PITCHED_MULT_ADD = 1,
    BSHIP_PITCHED_SCALAR = 2,
    BSHIP_PITCHED_UNARY = 3,
    BSHIP_PITCHED_DERIV = 4,
    BSHIP_PITCHED_CLIP = 5,
    BSHIP_PITCHED_COND = 6,
    BSHIP_PITCHED_FILL = 7
};
int bship_elementwise_pitched_f32(int family, int op, float s0, float s1,
                                  const float* a, int64_t a_row_stride, int a_col_stride,
                                  const float* b, int64_t b_row_stride, int b_col_stride,
                                  float* out, int64_t ld_out, int64_t rows, int64_t cols);

/* ------------------------------ reductions ------------------------------- */

/* sum_t (numpy 268-273, pycuda 375-381) of a (M,N): axis 0 -> out[N],
 * axis 1 -> out[M], axis -1 (None) -> out[1]. Deterministic (no float atomics). */
int bship_sum_f32(const float* a, float* out, int64_t M, int64_t N, int axis);
/* The same for a row-pitched a: ld_a elements from one row to the next (>= N).
 * out is dense. With ld_a == N this is bship_sum_f32. */
int bship_sum_pitched_f32(const float* a, int64_t ld_a, float* out, int64_t M, int64_t N, int axis);
/* bship_sum_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart
 * in the reference. Same kernels and the same bits as bship_sum_f32, but the partial
 * sums of the first stage go to a static 1 MiB device buffer (262144 floats, one per
 * device, held until the process ends) instead of a pool block, and the call makes no
 * hipMalloc/hipFree. A shape whose partial sums do not fit is refused with
 * BSHIP_ERR_BAD_DIMENSION; with the default launch shapes a dense matrix needs at most
 * 196608 floats (axis 0) or 2048 (axis -1), axis 1 needs none. All calls on a device
 * share the buffer: calls that overlap on one device (several streams, several host
 * threads) race; nothing in it needs clearing between calls (every partial sum read by
 * the second stage was written by the first stage of the same call). */
int bship_sum_noalloc_f32(const float* a, float* out, int64_t M, int64_t N, int axis);
/* softmax_m (numpy 292-295, pycuda 403-408): row-wise, one pass over HBM. */
int bship_softmax_rows_f32(const float* m, float* out, int64_t M, int64_t N);
/* The same for row-pitched m and out (ld_m, ld_out elements from one row to the next, >= N). */
int bship_softmax_rows_pitched_f32(const float* m, int64_t ld_m, float* out, int64_t ld_out,
                                   int64_t M, int64_t N);
/* is_fully_finite (numpy 69-70, pycuda 111-114). *result_host = 1 if every
 * element is finite. Blocks. */
int bship_isfinite_f32(const float* a, size_t n, int* result_host);

/* ------------------------------- indexing -------------------------------- */

/* binarize_v (numpy 99-101, pycuda 163-164): out[i,j] = (j == (int)v[i]) */
int bship_binarize_f32(const float* v, float* out, int64_t M, int64_t K);
/* The same with the labels ld_v elements apart (a column of a wider matrix) and a row-pitched out. */
int bship_binarize_pitched_f32(const float* v, int64_t ld_v, float* out, int64_t ld_out, int64_t M, int64_t K);
/* index_m_by_v (numpy 202-203, pycuda 284-285): out[i] = m[i, (int)v[i]].
 * Labels outside [0,K) are undefined in the reference; here they read as 0. */
int bship_index_m_by_v_f32(const float* m, const float* v, float* out,
                           int64_t M, int64_t K);
/* The same for a row-pitched m, and labels / results that are columns of wider matrices
 * (ld_v, ld_out elements from one row to the next). */
int bship_index_m_by_v_pitched_f32(const float* m, int64_t ld_m, const float* v, int64_t ld_v,
                                   float* out, int64_t ld_out, int64_t M, int64_t K);

/* --------------------------------- RNG ----------------------------------- */

/* Generators: every handler object owns a random stream (`self.rnd`, numpy 21;
 * randomness.py 10-80). bship_rng_create makes a new, unseeded generator;
 * bship_rng_select makes it the one that bship_rng_seed, bship_rng_get_state, the
 * mask draws, bship_fill_gaussian_f32 and the fast stream's calls use from then on
 * (nothing happens if it is selected already; otherwise masks drawn ahead for the
 * generator selected so far are given up, so every generator's stream stays the
 * sequential one). A recorded step draws from the generator that was selected
 * while it was recorded and selects it on every replay. Generator 0 exists from
 * the start and is selected until another one is. bship_rng_destroy frees a
 * generator's device state (generator 0 cannot be destroyed). */
int bship_rng_create(int* generator_id);
int bship_rng_select(int generator_id);
int bship_rng_destroy(int generator_id);
/* Seeds the selected generator's device-resident MT19937 state the way
 * numpy.random.RandomState(seed) does (randomness.py 66-80, numpy 21). Blocks. */
int bship_rng_seed(uint32_t seed);
/* generate_probability_mask (numpy 199-200): mask = (uniform[0,1) < p), drawing
 * the same 53-bit doubles, in the same order, as RandomState.uniform. */
int bship_prob_mask_f32(float* mask, size_t n, double p);
/* The same mask, written to a (rows, cols) matrix whose rows lie ld_mask elements apart
 * (a feature slice of a wider hub): element i of the draw goes to row i / cols, column
 * i % cols, exactly what `mask[:] = (uniform(size=shape) < p)` does on a strided view. */
int bship_prob_mask_pitched_f32(float* mask, int64_t ld_mask, int64_t rows, int64_t cols, double p);
/* fill_gaussian (numpy 193-194): out = std*standard_normal + mean with the
 * legacy polar method of RandomState.standard_normal. Blocks. */
int bship_fill_gaussian_f32(float* out, size_t n, double mean, double std);
/* Copies the 624 state words, position, has_gauss flag and cached gaussian to
 * the host (for tests and for saving the stream position). Blocks. */
int bship_rng_get_state(uint32_t* key_host, int* pos_host, int* has_gauss_host,
                        double* gauss_host);
/* The same operations on a named generator: what `handler.rnd` is to one handler object
 * (numpy 21, 193-200; randomness.py 66-80). The generator is selected and used under one lock,
 * so handlers that are driven from different threads cannot come between each other's selection
 * and draw. */
int bship_rng_seed_on(int generator, uint32_t seed);
int bship_rng_get_state_on(int generator, uint32_t* key_host, int* pos_host, int* has_gauss_host,
                           double* gauss_host);
int bship_prob_mask_on_f32(int generator, float* mask, size_t n, double p);
int bship_prob_mask_pitched_on_f32(int generator, float* mask, int64_t ld_mask, int64_t rows, int64_t cols,
                                   double p);
int bship_fill_gaussian_on_f32(int generator, float* out, size_t n, double mean, double std);

/* -------------------------------- dense ---------------------------------- */

/* dot_mm / dot_add_mm (numpy 176-185, pycuda 259-267): row-major
 * C(MxN) = alpha * op(A) * op(B) + beta * C through hipBLASLt.
 * op(A) is MxK: A is stored MxK (transa == 0) or KxM (transa != 0); ld* are
 * row pitches in elements. */
int bship_gemm_f32(int transa, int transb, int64_t M, int64_t N, int64_t K,
                   float alpha, const float* A, int64_t lda, const float* B,
                   int64_t ldb, float beta, float* C, int64_t ldc);
/* The product and bias of conv2d_forward_batch (numpy 149-171: out[i] = col . W^T,
 * then outputs += bias) in one call: C(M,N) = op(A) op(B) + bias, bias N elements,
 * one per column of C, added to the float32 accumulator in the product's epilogue
 * (the same single rounding as a separate add_mv over the stored product). */
int bship_gemm_bias_f32(int transa, int transb, int64_t M, int64_t N, int64_t K,
                        const float* A, int64_t lda, const float* B, int64_t ldb,
                        const float* bias, float* C, int64_t ldc);

/* conv2d_forward_batch (numpy 149-171) without the col matrix, for thin filters: stride 1, any
 * padding, kh*kw*c <= 128, f a multiple of 16 up to 64 (the first layer of an image network).
 * in: n images of (h, w, c), in_pitch floats apart; weights (f, kh, kw, c); bias (f); out (n, out_h,
 * out_w, f) dense. A workgroup stages the image rows of a band of output rows in LDS and the matrix
 * cores read the filter windows out of that copy. Any other geometry: BSHIP_ERR_UNSUPPORTED with
 * nothing launched (the caller then runs bship_im2col_nhwc_f32 + bship_gemm_bias_f32). Products sum
 * in k order in float32: equal to the im2col path up to the summation order. */
int bship_conv2d_fwd_thin_f32(const float* in, int64_t in_pitch, const float* weights,
                              const float* bias, float* out, int64_t n, int h, int w, int c, int f,
                              int kh, int kw, int pad, int stride_h, int stride_w);

/* conv2d_backward_batch (numpy 110-147) without the col matrix, for the same thin filters (and
 * kh*kw*c <= 127, a row of out_deltas times f within 4096 floats): weight_deltas (f, kh, kw, c) and
 * bias_deltas (f) are overwritten, in_deltas (n images of (h, w, c), in_deltas_pitch floats apart)
 * accumulated; out_deltas (n, out_h, out_w, f) dense. Three launches: the weights' and the bias's
 * deltas as per-workgroup partial sums over bands of images (the matrix cores read the filter
 * windows out of a copy of the image rows in LDS; the bias is a window entry that is always one),
 * their sum in workgroup order, and the inputs' deltas (out_deltas x weights into LDS per band, every
 * element of in_deltas adding the entries that fall on it in a fixed order: no atomics, the same
 * bits every time). Any other geometry: BSHIP_ERR_UNSUPPORTED with nothing launched. */
int bship_conv2d_bwd_thin_f32(const float* in, int64_t in_pitch, const float* weights,
                              const float* out_deltas, float* in_deltas, int64_t in_deltas_pitch,
                              float* weight_deltas, float* bias_deltas, int64_t n, int h, int w,
                              int c, int f, int kh, int kw, int pad, int stride_h, int stride_w);

/* im2col of a whole NHWC batch (_cpuop 251-277 applied per image by numpy
 * 158-166): col is (n*out_h*out_w, kh*kw*c). */
int bship_im2col_nhwc_f32(const float* in, float* col, int64_t n, int h, int w,
                          int c, int kh, int kw, int pad, int stride_h,
                          int stride_w);
/* col2im (_cpuop 282-309 applied per image by numpy 142-147): in_deltas +=
 * scatter of col, summed in the reference's (out_y, out_x) scan order. */
int bship_col2im_nhwc_f32(const float* col, float* in_deltas, int64_t n, int h,
                          int w, int c, int kh, int kw, int pad, int stride_h,
                          int stride_w);

/* maxpool2d_forward_batch (numpy 216-219, _cpuop 27-80). argmax holds the
 * per-image flat (y*w+x)*c+ch index as float32, -1 for an empty window. */
int bship_maxpool_fwd_nhwc_f32(const float* in, float* out, float* argmax,
                               int64_t n, int h, int w, int c, int out_h,
                               int out_w, int pool_h, int pool_w, int pad,
                               int stride_h, int stride_w);
/* maxpool2d_backward_batch (numpy 210-214, _cpuop 84-115); gather form that
 * adds in the reference's scan order, so the result is deterministic. */
int bship_maxpool_bwd_nhwc_f32(const float* argmax, const float* out_deltas,
                               float* in_deltas, int64_t n, int h, int w, int c,
                               int out_h, int out_w, int pool_h, int pool_w,
                               int pad, int stride_h, int stride_w);
/* avgpool2d_forward_batch (numpy 94-97, _cpuop 120-162) */
int bship_avgpool_fwd_nhwc_f32(const float* in, float* out, int64_t n, int h,
                               int w, int c, int out_h, int out_w, int pool_h,
                               int pool_w, int pad, int stride_h, int stride_w);
/* avgpool2d_backward_batch (numpy 89-92, _cpuop 167-202) */
int bship_avgpool_bwd_nhwc_f32(const float* out_deltas, float* in_deltas,
                               int64_t n, int h, int w, int c, int out_h,
                               int out_w, int pool_h, int pool_w, int pad,
                               int stride_h, int stride_w);

/* The forward recurrence of a peephole LSTM layer for all time steps in one launch
 * (lstm_layer.py 115-145: per time step the four recurrent products y[t-1] R^T accumulated into
 * Za, Ia, Fa, Oa, then the elementwise part that bship_lstm_fwd_step_f32 does). On entry Za, Ia,
 * Fa, Oa hold the input products x W^T (lstm_layer.py 110-113). Every array of the first group is
 * (time_steps + 1, batch, n), dense; slab `time_steps` is the context slot that y[t-1] and
 * Ca[t-1] mean at t = 0. R_all is the stacked (4n, n) matrix [Rz; Ri; Rf; Ro] (the four matrices
 * are adjacent in the layer's parameter vector). The recurrent weights stay in LDS for the whole
 * sequence, one workgroup per 4 hidden units on a compute unit of its own (a batch above 64 rows
 * is two row sets of four wavefronts each in the same workgroup), and the workgroups meet at one
 * grid barrier per time step whose wait is bounded (BSHIP_GRID_BARRIER_SPINS polls, default 2^21;
 * a value that is not a whole number is ignored, and 0 is kept as the test hook that makes every
 * barrier fail at once): if it runs out, e.g. because other work kept some workgroups off the device, every workgroup
 * exits, the call returns BSHIP_ERR_TIMEOUT and the buffers hold an unfinished pass. Needs
 * n % 4 == 0, batch <= 128, n <= 1024 and n / 4 workgroups resident together (one per compute
 * unit); otherwise BSHIP_ERR_UNSUPPORTED before anything is launched.
 * Takes 4 KB + 512 bytes per hidden unit and time step from the pool for the flags and the
 * transposed operand, one buffer per time step so that no cache ever holds a stale line of it;
 * beyond BSHIP_LSTM_SEQ_SCRATCH_MB (default 256) megabytes the buffers are reused in turn and
 * the caches are invalidated at every barrier instead.
 * Results equal the step-by-step path up to the summation order of the products. Blocks; not
 * recordable. */
int bship_lstm_fwd_sequence_f32(int act, int64_t time_steps, int64_t batch, int64_t n,
                                const float* R_all, float* Za, float* Zb, float* Ia, float* Ib,
                                float* Fa, float* Fb, float* Oa, float* Ob, float* Ca, float* Cb,
                                float* y, const float* pi, const float* pf, const float* po,
                                const float* bz, const float* bi, const float* bf, const float* bo);

/* bship_lstm_bwd_step_packed_f32 behind bship_dot_small_tn_f32 (batch <= 128): the recurrent deltas
 * packed[t+1] . [Rz;Ri;Rf;Ro] arrive as `parts` partial products (slabs of (batch, n), part_stride
 * floats apart, added in ascending order), dy receives deltas + their sum, and [dZa|dIa|dFa|dOa]
 * of this step leaves transposed: packed_t_out is (4n, 128), row g*n + j, column b; columns >= batch
 * are not written (allocate it zeroed). The arithmetic is lstm_layer.py 186-214, as in
 * bship_lstm_bwd_step_f32. */
int bship_lstm_bwd_step_thin_f32(int act, int64_t batch, int64_t n, const float* deltas, const float* dy_parts,
                                 int parts, int64_t part_stride, float* dy, float* packed_t_out, const float* Zb,
                                 const float* Ib, const float* Fb, const float* Ob, const float* Cb,
                                 const float* Ca_prev, const float* Fb_next, const float* dIa_next,
                                 const float* dFa_next, const float* dCa_next, float* dZa, float* dZb, float* dIa,
                                 float* dIb, float* dFa, float* dFb, float* dOa, float* dOb, float* dCa, float* dCb,
                                 const float* pi, const float* pf, const float* po);

/* Matrix product with a thin left operand that is stored transposed, for the per-time-step
 * recurrent products of lstm_layer.py 115-145 and 180-205 (dot_mm / dot_add_mm of a (batch, n)
 * slab, numpy_handler.py 211-229, with batch <= 128):
 *     c[s] (M x N, row pitch ldc) = A[:, K-range s] . b[K-range s, :]     for s = 0 .. splits-1
 * where aT holds A transposed: K rows of 128 floats, element (k, i) = A[i][k], columns >= M zero,
 * 16-byte aligned; b is (K, N) with row pitch ldb. splits > 1 cuts K into that many ranges of whole
 * 16-blocks whose results go to the slabs c + s * c_split_stride (floats), for the caller to add in
 * a fixed order; splits == 1 writes the whole product to c. Sums run over k in ascending blocks per
 * wavefront quarter, ((q0 + q1) + (q2 + q3)): equal to a float32 BLAS product up to summation order.
 * M > 128 or operands of 1 GiB and more: BSHIP_ERR_UNSUPPORTED. Recordable. */
int bship_dot_small_tn_f32(const float* aT, const float* b, float* c, int64_t M, int64_t N, int64_t K,
                           int64_t ldb, int64_t ldc, int splits, int64_t c_split_stride);

/* dst[c][r] = src[r][c] for r < rows, c < cols (row pitches ld_src >= cols, ld_dst >= rows);
 * columns >= rows of dst are left as they are. Produces the transposed operands of
 * bship_dot_small_tn_f32 (ld_dst = 128) and transposed weight matrices. No counterpart in
 * base_handler.py: NumPy callers write a.T. */
int bship_transpose_f32(const float* src, int64_t rows, int64_t cols, int64_t ld_src, float* dst,
                        int64_t ld_dst);

/* The image operations on image-pitched arrays. A layer whose input or output is
 * a feature slice of a hub that several layers share (buffer_structure.py
 * 232-245) sees images that are contiguous (h*w*c elements) but lie a pitch of
 * the hub's full feature count apart; NumpyHandler's _cpuop routines take such
 * strided views as they are. Every *_pitch is the number of elements from one
 * image to the next in that array (at least the image size; the image size
 * itself gives the dense functions above). col stays dense. */
int bship_im2col_nhwc_pitched_f32(const float* in, int64_t in_pitch, float* col, int64_t n,
                                  int h, int w, int c, int kh, int kw, int pad,
                                  int stride_h, int stride_w);
int bship_col2im_nhwc_pitched_f32(const float* col, float* in_deltas, int64_t in_deltas_pitch,
                                  int64_t n, int h, int w, int c, int kh, int kw, int pad,
                                  int stride_h, int stride_w);
int bship_maxpool_fwd_nhwc_pitched_f32(const float* in, int64_t in_pitch, float* out,
                                       int64_t out_pitch, float* argmax, int64_t argmax_pitch,
                                       int64_t n, int h, int w, int c, int out_h, int out_w,
                                       int pool_h, int pool_w, int pad, int stride_h,
                                       int stride_w);
int bship_maxpool_bwd_nhwc_pitched_f32(const float* argmax, int64_t argmax_pitch,
                                       const float* out_deltas, int64_t out_deltas_pitch,
                                       float* in_deltas, int64_t in_deltas_pitch, int64_t n,
                                       int h, int w, int c, int out_h, int out_w, int pool_h,
                                       int pool_w, int pad, int stride_h, int stride_w);
int bship_avgpool_fwd_nhwc_pitched_f32(const float* in, int64_t in_pitch, float* out,
                                       int64_t out_pitch, int64_t n, int h, int w, int c,
                                       int out_h, int out_w, int pool_h, int pool_w, int pad,
                                       int stride_h, int stride_w);
int bship_avgpool_bwd_nhwc_pitched_f32(const float* out_deltas, int64_t out_deltas_pitch,
                                       float* in_deltas, int64_t in_deltas_pitch, int64_t n,
                                       int h, int w, int c, int out_h, int out_w, int pool_h,
                                       int pool_w, int pad, int stride_h, int stride_w);

/* --------------------------- fused layer steps --------------------------- */

/* Extensions beyond the handler interface: one launch for the elementwise
 * part of one LSTM time step, chaining the same float32 operations in the
 * order the layer issues them as single handler calls, so the results are
 * bit-identical to that sequence. All matrices are (batch, n) dense; the
 * peephole vectors p* and the biases b* hold n elements.
 * Activation codes: the act_func table of base_handler.py 57-63. */
enum {
    BSHIP_ACT_SIGMOID = 0,
    BSHIP_ACT_TANH = 1,
    BSHIP_ACT_REL = 2,
    BSHIP_ACT_LINEAR = 3,
    BSHIP_ACT_EL = 4
};
/* LstmLayerImpl.forward_pass, the part of the loop body after the four
 * dot_add_mm calls (lstm_layer.py 121-145). Za, Ia, Fa, Oa hold the
 * accumulated products on entry and the biased pre-activations on return. */
int bship_lstm_fwd_step_f32(int act, int64_t batch, int64_t n, float* Za,
                            float* Zb, float* Ia, float* Ib, float* Fa,
                            float* Fb, float* Oa, float* Ob, float* Ca,
                            float* Cb, const float* Ca_prev, float* y,
                            const float* pi, const float* pf, const float* po,
                            const float* bz, const float* bi, const float* bf,
                            const float* bo);
/* LstmLayerImpl.backward_pass, the part of the loop body between the
 * recurrent dot_add_mm calls into dy and the dot_add_mm calls that follow
 * (lstm_layer.py 186-214). dCa holds its initial content on entry (the layer
 * accumulates into it); the *_next arguments are the buffers of time t+1. */
int bship_lstm_bwd_step_f32(int act, int64_t batch, int64_t n, const float* dy,
                            const float* Zb, const float* Ib, const float* Fb,
                            const float* Ob, const float* Cb,
                            const float* Ca_prev, const float* Fb_next,
                            const float* dIa_next, const float* dFa_next,
                            const float* dCa_next, float* dZa, float* dZb,
                            float* dIa, float* dIb, float* dFa, float* dFb,
                            float* dOa, float* dOb, float* dCa, float* dCb,
                            const float* pi, const float* pf, const float* po);
/* The same two steps for a caller that forms the four recurrent products of a
 * time step as ONE matrix product over the stacked recurrent weights
 * [Rz;Ri;Rf;Ro] (4n x n, as they lie in brainstorm's parameter vector,
 * lstm_layer.py 62-65) instead of four accumulating ones:
 *  - forward: rec (batch, 4n) = y[t-1] [Rz;Ri;Rf;Ro]^T, columns [z|i|f|o], is
 *    added to Za, Ia, Fa, Oa before the step proper;
 *  - backward: dy holds packed[t+1] [Rz;Ri;Rf;Ro] on entry and receives
 *    deltas + that (lstm_layer.py 181-185); packed_out (batch, 4n) receives
 *    [dZa|dIa|dFa|dOa] of this step, the left operand of the next product.
 *    deltas may be NULL: dy is then complete on entry (bship_lstm_bwd_step_f32's
 *    meaning) and the call only adds the packed copy of the step's gate deltas.
 * The elementwise arithmetic is the same; the matrix products sum in another
 * order than four separate ones, so results agree to rounding, not bit for bit. */
int bship_lstm_fwd_step_packed_f32(int act, int64_t batch, int64_t n,
                                   const float* rec, float* Za, float* Zb,
                                   float* Ia, float* Ib, float* Fa, float* Fb,
                                   float* Oa, float* Ob, float* Ca, float* Cb,
                                   const float* Ca_prev, float* y,
                                   const float* pi, const float* pf,
                                   const float* po, const float* bz,
                                   const float* bi, const float* bf,
                                   const float* bo);
int bship_lstm_bwd_step_packed_f32(int act, int64_t batch, int64_t n,
                                   const float* deltas, float* dy,
                                   float* packed_out, const float* Zb,
                                   const float* Ib, const float* Fb,
                                   const float* Ob, const float* Cb,
                                   const float* Ca_prev, const float* Fb_next,
                                   const float* dIa_next, const float* dFa_next,
                                   const float* dCa_next, float* dZa, float* dZb,
                                   float* dIa, float* dIb, float* dFa,
                                   float* dFb, float* dOa, float* dOb,
                                   float* dCa, float* dCb, const float* pi,
                                   const float* pf, const float* po);

/* SoftmaxCELayerImpl.forward_pass (softmax_ce_layer.py 79-89): softmax_m(inputs, probs), then in one
 * launch loss[i] = -log(clip(probs[i, int(targets[i])], 1e-6, 1)) (index_m_by_v, clip_t, log_t,
 * mult_st with the same roundings). inputs, probs are (M, K); targets, loss (M, 1). */
int bship_softmax_ce_fwd_f32(const float* inputs, const float* targets, float* probs, float* loss,
                             int64_t M, int64_t K);
/* SoftmaxCELayerImpl.backward_pass (softmax_ce_layer.py 108-112) in one pass: t_bin = onehot(targets);
 * t_bin = -1 * t_bin; t_bin += probs; t_bin *= dloss (a column); dinputs = t_bin + dinputs. */
int bship_softmax_ce_bwd_f32(const float* probs, const float* targets, const float* dloss, float* t_bin,
                             float* dinputs, int64_t M, int64_t K);
/* MomentumStepper.run after the passes (steppers.py 104-112) in one pass: velocity = momentum * velocity;
 * velocity += neg_learning_rate * gradients; parameters = velocity + parameters. */
int bship_momentum_update_f32(float momentum, float neg_learning_rate, const float* gradients,
                              float* velocity, float* parameters, size_t n);

/* HighwayLayerImpl.forward_pass (highway_layer.py 48-51) in one pass:
 * tmp = H - x; tmp = T * tmp; y = tmp + x. */
int bship_highway_fwd_f32(const float* H, const float* T, const float* x,
                          float* y, size_t n);
/* HighwayLayerImpl.backward_pass (highway_layer.py 64-71) in one pass:
 * dx += (1 - T) * dy; dH += T * dy; dT += (H - x) * dy. */
int bship_highway_bwd_f32(const float* H, const float* T, const float* x,
                          const float* dy, float* dx, float* dH, float* dT,
                          size_t n);
/* add_mv(outputs, bias, outputs) followed by inplace_act_func[act](outputs)
 * (fully_connected_layer.py 61-62) in one pass: out = act(in + bias), in and
 * out (M,N), bias N elements, act one of BSHIP_ACT_*. out may be in. */
int bship_bias_act_f32(int act, const float* in, const float* bias, float* out,
                       int64_t M, int64_t N);
/* DropoutLayerImpl.forward_pass, training branch (dropout_layer.py 41-45) in
 * one pass behind the mask: generate_probability_mask(mask, keep_probability);
 * out = in * mask; out = scale * out. The mask comes from the same stream, at
 * the same position, as bship_prob_mask_f32 would draw it. */
int bship_dropout_fwd_f32(const float* in, float* mask, float* out, size_t n,
                          double keep_probability, float scale);
/* Optional fast mask stream. No counterpart in NumpyHandler: masks come from
 * the counter-based Philox4x32-10 generator (four mask elements per block, a
 * pure function of a 64-bit key and a 64-bit block number kept in device
 * memory), one parallel launch per mask instead of the sequential MT19937 walk.
 * For callers that want dropout at memory speed and do not need the masks
 * NumpyHandler would draw; the reference's GPU handler is in the same position
 * (cuRAND XORWOW, pycuda_handler.py 37-39 and 191-193). element i of a mask is
 * 1.0 when word i%4 of block next_block + i/4 is below floor(p * 2^32); every
 * call advances next_block by ceil(n/4), also inside recorded steps.
 * bship_dropout_fwd_fast_f32 is bship_dropout_fwd_f32 on this stream. */
int bship_fast_rng_seed(unsigned long long seed);
int bship_fast_rng_get_state(unsigned long long* seed_host, unsigned long long* next_block_host);
int bship_prob_mask_fast_f32(float* mask, size_t n, double p);
int bship_dropout_fwd_fast_f32(const float* in, float* mask, float* out, size_t n,
                               double keep_probability, float scale);
/* The dropout pass and the fast stream's calls on a named generator (see bship_rng_seed_on). */
int bship_dropout_fwd_on_f32(int generator, const float* in, float* mask, float* out, size_t n,
                             double keep_probability, float scale);
int bship_fast_rng_seed_on(int generator, unsigned long long seed);
int bship_fast_rng_get_state_on(int generator, unsigned long long* seed_host,
                                unsigned long long* next_block_host);
int bship_prob_mask_fast_on_f32(int generator, float* mask, size_t n, double p);
int bship_dropout_fwd_fast_on_f32(int generator, const float* in, float* mask, float* out, size_t n,
                                  double keep_probability, float scale);
/* BatchNormLayerImpl.forward_pass (batch_normalization_layer.py 54-105) on
 * (M,N) matrices and N-element vectors. training != 0: batch statistics (the
 * negative batch mean and then the deviation go through sigma_b as in the
 * layer), running averages mu and sigma updated with `decay`, three passes
 * over the matrix instead of seven: column sums; centering fused with the
 * column sums of squares; normalise + scale + shift. training == 0: one pass
 * with the running mu and sigma. decay and epsilon arrive as the Python floats
 * (the layer computes 1.0 - decay in double before the handler rounds it). */
int bship_batchnorm_fwd_f32(int training, const float* inputs,
                            const float* gamma, const float* beta, float* mu,
                            float* sigma, double decay, double epsilon,
                            float* sigma_b, float* centered, float* x_hat,
                            float* out, int64_t M, int64_t N);
/* BatchNormLayerImpl.backward_pass (batch_normalization_layer.py 107-152):
 * dgamma += colsum(out_deltas * x_hat); dbeta += colsum(out_deltas);
 * in_deltas += ((out_deltas - x_hat * dgamma_b / M) - dbeta_b / M) * gamma / sigma_b
 * with the layer's order of float32 operations. Takes 3 N-element temporaries
 * from the pool. */
int bship_batchnorm_bwd_f32(const float* out_deltas, const float* x_hat,
                            const float* gamma, const float* sigma_b,
                            float* dgamma, float* dbeta, float* in_deltas,
                            int64_t M, int64_t N);

/* ---------------------------- the fusing window --------------------------- */

/* brainstorm's layers know the primitive operations only: an LSTM time step is 19 handler calls
 * (lstm_layer.py 117-145), a batch normalisation pass 15 (batch_normalization_layer.py 68-105).
 * With the fusing window on, the entry points of the elementwise, matrix-vector, fill, dense sum,
 * softmax, one-hot, gather and dense mask operations do not launch at once: a call is held back
 * while the calls so far are the beginning of one of the layers' sequences (LSTM forward and
 * backward step, bias + activation, dropout, softmax cross entropy forward and backward, momentum
 * update, Highway forward and backward, batch normalisation forward, inference and backward:
 * same operations, same operand identities), a complete sequence is enqueued as the fused entry
 * point that computes it (same float32 operations in the same order: same bits in every array the
 * sequence writes), and everything else is enqueued as it was called, in call order. Arrays that
 * a sequence only uses as temporaries (highway_layer.py 48 and 64, batch_normalization_layer.py
 * 119-120) are not written by the fused kernels: such a sequence is fused only when bship_free
 * of the temporaries follows its last call directly, as it does when the layer drops them.
 * Matrix products are never held; they overtake held calls that share no operand with them which
 * either side writes. Every other entry point (copies to the host, bship_sync, allocation,
 * recording, ...) first enqueues what is held. Errors of a held call are reported by the call that
 * causes it to be enqueued. The switch belongs to the library, not to a handler object.
 * mode 0: off. mode 1: as described (same bits as mode 0). mode 2 ("stacked") additionally holds
 * the matrix products and copies of an LSTM time step (lstm_layer.py:117-145, 173-205): the four
 * recurrent products of a step, whose weight matrices lie back to back in brainstorm's parameter
 * vector, run as ONE product over the stacked matrix [Rz;Ri;Rf;Ro] (forward: into a scratch matrix
 * that the step kernel adds; backward: from a packed copy of the previous step's gate deltas that
 * the step kernel leaves behind), which is what bship_lstm_*_step_packed_f32 offer a handler-aware
 * caller. The products then sum in another order, so results agree with modes 0 and 1 to rounding
 * (1e-6 relative), not bit for bit. */
int bship_fusing_set(int mode);
int bship_fusing_get(int* on_host);
/* Enqueues what the window holds. */
int bship_fusing_flush(void);
/* Counters since the last reset: operations that entered the window, those enqueued as they were,
 * those replaced by fused launches, fused launches, matrix products that overtook held calls. */
int bship_fusing_stats(unsigned long long* calls, unsigned long long* unfused,
                       unsigned long long* fused_calls, unsigned long long* fused_launches,
                       unsigned long long* overtaken, int reset);

#ifdef __cplusplus
}
#endif
#endif /* BSHIP_H */
