/*
 * tftq -- FP8 (OCP e4m3fn) quantized-collective kernels for AMD MI355X (gfx950).
 *
 * C ABI of libtftq.so.  Plain pointers and sizes only; no torch types.
 * The three compute entry points replace the three launchers of the reference
 * (torchft/quantization.py): fused_quantize_into_fp8 (:531-588),
 * fused_reduce_fp8 (:638-686) and fused_dequantize_from_fp8 (:591-635).
 * The plan replaces _prepare_quantize_fp8 (:431-528).
 *
 * Conventions
 *  - every function returns 0 on success; a negative value is a TFTQ_E_* code,
 *    a positive value is a hipError_t.  Nothing aborts or throws.
 *  - a plan describes shapes, strides, element type and group size only.  It
 *    holds no address and belongs to no device: tensor addresses, the packed
 *    buffer, the device and the stream are arguments of every compute call.
 *  - `device` is the ordinal of the device that all device addresses of the
 *    call belong to; the library makes it current for the duration of the
 *    call and restores the caller's device before it returns.  -1 = the device
 *    that is current on the calling thread.
 *  - kernels are enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *    null stream) and the host is never synchronised.
 *  - functions are thread-safe; a plan is immutable and may be used from
 *    several threads, devices and streams at once.
 *  - the library allocates no device memory.  Lists of up to TFTQ_N_INLINE
 *    tensors need none beyond tensors and packed buffer (their descriptors
 *    travel in the kernel arguments); longer lists need two caller-owned device
 *    buffers, see "Long lists" below.
 *
 * Packed buffer (byte-for-byte the reference's, quantization.py:108-123,
 * 495-503), for tensor i of shape [m_i, n_i] and group size ws:
 *    row_bytes_i  = (ceil(n_i / 4) + 1) * 4
 *    slice_rows_i = ceil(m_i / ws)
 *    slot_off_i   = sum_{j<i} slice_rows_j * row_bytes_j
 *    slot_size    = sum_i slice_rows_i * row_bytes_i
 *    output_size  = ws * slot_size
 *    addr(i, r)   = (r / slice_rows_i) * slot_size + slot_off_i
 *                   + (r % slice_rows_i) * row_bytes_i
 *    at addr: [fp32 scale][n_i e4m3fn codes][zero padding to row_bytes_i]
 */
#ifndef TFTQ_H
#define TFTQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TFTQ_VERSION 2

/* element types of the tensors being (de)quantized (quantization.py:474-478) */
#define TFTQ_F32 0
#define TFTQ_F16 1
#define TFTQ_BF16 2

/* lists of at most this many tensors need no device memory for their descriptors */
#define TFTQ_N_INLINE 16

/* error codes (negative); positive return values are hipError_t */
#define TFTQ_E_ARG (-1)      /* bad argument (null pointer, ws <= 0, rank out of range ...) */
#define TFTQ_E_DTYPE (-2)    /* "Only fp32, fp16 and bf16 are supported" (:474-478) */
#define TFTQ_E_SHAPE (-3)    /* negative or too large dimension */
#define TFTQ_E_SIZE (-4)     /* "Output size does not match" (:621, :672) */
#define TFTQ_E_NOMEM (-5)    /* host allocation failed */
#define TFTQ_E_NOTABLE (-6)  /* a list longer than TFTQ_N_INLINE needs `table` (and `pointers`) */
#define TFTQ_E_ARCH (-7)     /* the device is not gfx950 */
#define TFTQ_E_TOOBIG (-8)   /* tftq_reduce_static: the list's table exceeds TFTQ_STATIC_TABLE_BYTES */
#define TFTQ_E_BUSY (-9)     /* tftq_reduce_static: a call on another stream of the device has not finished */

typedef struct tftq_plan tftq_plan;

/* library version (TFTQ_VERSION of the build) */
int tftq_version(void);

/* Identifies the sources the library was built from (a hash that the build passes in;
 * "unknown" without one).  Static storage. */
const char *tftq_build_id(void);

/* Text for a return value of this library (static storage). */
const char *tftq_strerror(int code);

/* 0 when device `device` (-1: the current one) can run the kernels (gfx950), else
 * TFTQ_E_ARCH or a hipError_t. */
int tftq_check_device(int device);

/*
 * Layout arithmetic of _prepare_quantize_fp8 (quantization.py:486-503), host
 * only.  shapes: [n_tensors][2] = (m, n); 1-D tensors are passed as (k, 1)
 * (:487-488).  slot_off (may be NULL) receives n_tensors byte offsets.
 */
int tftq_layout(int n_tensors, const int64_t *shapes, int ws, int64_t *slot_off,
                int64_t *slot_size, int64_t *output_size);

/*
 * Builds the work plan for one list of tensors: the layout above plus the
 * partition of all rows into workgroups for the three kernels.  Replaces the
 * shape, stride and offset tables that _prepare_quantize_fp8 uploads on every
 * call (quantization.py:505-515); the addresses (its fourth table) are an
 * argument of the compute calls.  Host only, no HIP call.
 *   dtype    TFTQ_F32 / TFTQ_F16 / TFTQ_BF16
 *   shapes   [n_tensors][2] (m, n)
 *   strides  [n_tensors][2] element strides (row, column); any values
 */
int tftq_plan_create(int dtype, int n_tensors, const int64_t *shapes, const int64_t *strides,
                     int ws, tftq_plan **out);
void tftq_plan_destroy(tftq_plan *plan);

int64_t tftq_plan_output_size(const tftq_plan *plan); /* bytes of the packed buffer */
int64_t tftq_plan_slot_size(const tftq_plan *plan);   /* output_size / ws */
int64_t tftq_plan_max_rows(const tftq_plan *plan);    /* i_max_row_num of the reference */
int tftq_plan_n_tensors(const tftq_plan *plan);

/*
 * Long lists (more than TFTQ_N_INLINE tensors).  The kernels read the
 * descriptors from device memory that the caller owns:
 *   table     tftq_plan_table_bytes() bytes, 256-byte aligned, holding a copy of
 *             tftq_plan_table_host(): descriptors and lookup index, no addresses.
 *             The same image serves every device, stream and list of tensors of
 *             these shapes; copy it once per device, any way you like, before
 *             the first kernel that uses it runs.
 *   pointers  8 * n_tensors bytes, 8-byte aligned: the tensors' addresses.  When a
 *             compute call is given `tensors` (host array), it first writes them
 *             here with small kernels on `stream` (the host array is read
 *             before the call returns; nothing blocks); with tensors == NULL it
 *             uses what `pointers` already holds.  One `pointers` buffer must
 *             not be written by calls that overlap in time.  All arguments are
 *             checked before the addresses are written; a call whose kernel launch
 *             then fails with a hipError_t has still rewritten `pointers`.
 * For short lists both are ignored (pass NULL) and tftq_plan_table_bytes() is 0.
 */
int64_t tftq_plan_table_bytes(const tftq_plan *plan);
const void *tftq_plan_table_host(const tftq_plan *plan);

/* Writes the n_tensors addresses of `tensors` (host array) to `pointers` (device) on
 * `stream`: what the compute calls do when they are given `tensors` for a long list. */
int tftq_upload_pointers(const tftq_plan *plan, const void *const *tensors, void *pointers,
                         int device, void *stream);

/*
 * fused_quantize_into_fp8 (quantization.py:531-588).  Reads the tensors,
 * writes every byte of packed[0 .. output_size): scales, codes, zero padding
 * and zero padding rows, so `packed` needs no prior memset (the reference
 * relies on torch.zeros, :567-571).  packed must be 4-byte aligned.
 *   tensors  host array [n_tensors]: device address of element (0,0) of each
 *            tensor (may be NULL for a long list whose `pointers` are current)
 */
int tftq_quantize(const tftq_plan *plan, const void *const *tensors, const void *table,
                  void *pointers, void *packed, int64_t packed_bytes, int device, void *stream);

/*
 * fused_reduce_fp8 (quantization.py:638-686).  packed holds ws slots, slot p =
 * peer p's quantization of this rank's row slice.  Sums the slots in fp32 in
 * the order rank, rank+1, ... (wrapping, :405-407), requantizes and overwrites
 * slot `rank` (scale and codes of every row, padding rows included).  is_avg
 * != 0 divides by ws (:682).  No tensor is touched (the reference's launcher
 * ignores their addresses too, :675-686).
 */
int tftq_reduce(const tftq_plan *plan, const void *table, void *packed, int64_t packed_bytes,
                int rank, int is_avg, int device, void *stream);

/*
 * fused_dequantize_from_fp8 (quantization.py:591-635).  Writes
 * cast(float(code) / scale) into the tensors (all m_i real rows).
 */
int tftq_dequantize(const tftq_plan *plan, void *const *tensors, const void *table,
                    void *pointers, const void *packed, int64_t packed_bytes, int device,
                    void *stream);

/*
 * fused_dequantize_from_fp8 followed by the caller's normalisation of the result,
 * `tensor /= num_participants` in the continuation of Manager.allreduce
 * (manager.py:450-452), in one pass over the tensors instead of two.  Writes
 * cast(float(cast(float(code) / scale)) * post_scale): the value is rounded to
 * the tensors' dtype as tftq_dequantize stores it, widened again and multiplied
 * in fp32, which is what torch's division of a GPU tensor by a host scalar
 * computes with post_scale = (float)(1.0 / divisor).  The bytes equal those of
 * tftq_dequantize followed by that division.
 */
int tftq_dequantize_scaled(const tftq_plan *plan, void *const *tensors, const void *table,
                           void *pointers, const void *packed, int64_t packed_bytes,
                           float post_scale, int device, void *stream);

/*
 * tftq_reduce for callers that cannot hand over device memory for `table` and may not
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  For a long list the table image
 * is written, with small kernels on `stream`, into a fixed array of
 * TFTQ_STATIC_TABLE_BYTES bytes that the library's code object holds on every device
 * it runs on, and the reduce kernel reads it from there; lists whose table is larger
 * are refused with TFTQ_E_TOOBIG (90 to 190 bytes per tensor: lists of 2800 tensors always fit).
 * Short lists use no scratch memory at all.  The call allocates and frees nothing; it
 * costs one small kernel per 3584 bytes of table in front of the reduce kernel.  The
 * array's address on a device is looked up once, by tftq_check_device() for that device
 * or else by the first call there (which should then not run under stream capture).
 * All calls on one device share that array.  Calls on one stream are ordered by the stream.
 * A call on another stream than the last one, while the last one's kernel has not finished,
 * queues nothing and returns TFTQ_E_BUSY (wait for that stream, or make this one wait for it,
 * and call again); calls from several threads are taken one at a time.  Calls that a stream
 * capture records are not checked against each other or against later calls: replays of
 * graphs that hold such calls, and eager calls beside them, must be serialised by the
 * caller.  Results are those of tftq_reduce.
 */
#define TFTQ_STATIC_TABLE_BYTES (512 * 1024)
int tftq_reduce_static(const tftq_plan *plan, void *packed, int64_t packed_bytes, int rank,
                       int is_avg, int device, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TFTQ_H */
