// Streaming kernels without arithmetic: what HBM delivers on MI355X (gfx950) for
// the read : write mixes and access patterns of the three stages, measured by
// `bench.py --config ceiling` beside the product kernels.  Benchmark
// infrastructure: built into its own library (libtftq_ceiling.so), never loaded
// by torchft_amd.quantization.
//
// Plain mixes: a workgroup of 256 lanes moves one chunk the way the product
// kernels do, every lane issues all its loads back to back (8 in flight), then
// stores.  Sources and destinations are contiguous arrays, so neither row
// boundaries nor scales nor the lookup of a tensor cost anything.
//
//   kind     reads per lane   writes per lane   stage with this mix
//   RO       8 x 16 B         -                 (read bandwidth)
//   WO       -                8 x 16 B          (write bandwidth)
//   R2W1     8 x 16 B         8 x 8 B           quantize, 16-bit tensors
//   R1W2     8 x 8 B          8 x 16 B          dequantize, 16-bit tensors
//   R4W1     8 x 16 B         8 x 4 B           quantize, fp32 tensors
//   R1W4     8 x 4 B          8 x 16 B          dequantize, fp32 tensors
//   R8W1     8 x 16 B         1 x 16 B          reduce, 8 peers (one contiguous source)
//
// Patterns: the memory accesses of a product kernel and nothing else.
//
//   RED      reduce on rows of up to 4096 codes: one workgroup per row, a lane loads one
//            16-byte vector of each of 8 sources one slot apart (rows of row_bytes, payload
//            4 bytes behind the row start), the result goes over source `rank` in place
//   (k_reduce_pattern_mix, tftq_ceiling_reduce_mix: the same for a group of 4 and a slot of
//            two row lengths, the shape of the reduce of an fp32 pseudo-gradient)
//   RED_LINE RED with the 1 KB that a wavefront accesses moved down to a 128-byte line:
//            what it costs that packed rows start anywhere
//   DEQ      dequantize on 16-bit rows of 4096 columns: one wavefront per row, a lane loads
//            8 x 8 bytes of the packed row and stores 8 x 16 bytes of the 8 KB tensor row
//   QNT      quantize on 16-bit rows of 4096 columns: four rows per workgroup, one wavefront per
//            row, a lane loads 8 x 16 bytes of the 8 KB tensor row and produces 8 x 8 bytes of
//            the packed row of row_bytes.  nt_stores: the workgroup assembles its four packed
//            rows in LDS and writes them as whole lines with streaming stores, as the product
//            does; otherwise plain 8-byte stores straight from the registers.  Rows of one slot.
//
// `eighths` (patterns only): workgroup ids go round-robin to the 8 XCDs of the chip; with
// eighths XCD x works through the x-th contiguous eighth of the rows, without it workgroup
// b takes piece b (neighbouring pieces run on different XCDs at the same time).

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x2 u32x2_a4 __attribute__((aligned(4)));
#define GLOBAL __attribute__((address_space(1)))

enum { C_RO = 0, C_WO = 1, C_R2W1 = 2, C_R1W2 = 3, C_R4W1 = 4, C_R1W4 = 5, C_R8W1 = 6,
       C_RED = 7, C_RED_LINE = 8, C_DEQ = 9, C_QNT = 10,
       // the four mixes of quantize and dequantize with 4 steps per lane instead of 8
       C_R2W1_4 = 11, C_R1W2_4 = 12, C_R4W1_4 = 13, C_R1W4_4 = 14, C_KINDS = 15 };

template <typename V, bool NT>
__device__ __forceinline__ V ld(GLOBAL const V *p)
{
    return NT ? __builtin_nontemporal_load(p) : *p;
}
template <typename V, bool NT>
__device__ __forceinline__ void st(V v, GLOBAL V *p)
{
    if (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// RV / WV: bytes a lane reads / writes per step (STEPS steps per chunk: all its loads, then
// all its stores); WV == 2 stands for one 16-byte store per 8 loads.
template <int RV, int WV, bool NTL, bool NTS, int STEPS = 8>
__global__ __launch_bounds__(256) void k_stream(const uint8_t *src, uint8_t *dst, int64_t chunks, u32 never)
{
    const int64_t c = blockIdx.x;
    if (c >= chunks) return;
    const int t = threadIdx.x;
    u32 x[STEPS][4];
#pragma unroll
    for (int k = 0; k < STEPS; k++) x[k][0] = x[k][1] = x[k][2] = x[k][3] = (u32)t + k;
    if constexpr (RV == 16) {
        GLOBAL const u32x4 *s = (GLOBAL const u32x4 *)(uint64_t)(src + c * (STEPS * 256 * 16));
#pragma unroll
        for (int k = 0; k < STEPS; k++) {
            const u32x4 v = ld<u32x4, NTL>(s + k * 256 + t);
            x[k][0] = v.x; x[k][1] = v.y; x[k][2] = v.z; x[k][3] = v.w;
        }
    } else if constexpr (RV == 8) {
        GLOBAL const u32x2 *s = (GLOBAL const u32x2 *)(uint64_t)(src + c * (STEPS * 256 * 8));
#pragma unroll
        for (int k = 0; k < STEPS; k++) {
            const u32x2 v = ld<u32x2, NTL>(s + k * 256 + t);
            x[k][0] = v.x; x[k][1] = v.y; x[k][2] = v.x ^ 1u; x[k][3] = v.y ^ 1u;
        }
    } else if constexpr (RV == 4) {
        GLOBAL const u32 *s = (GLOBAL const u32 *)(uint64_t)(src + c * (STEPS * 256 * 4));
#pragma unroll
        for (int k = 0; k < STEPS; k++) {
            const u32 v = ld<u32, NTL>(s + k * 256 + t);
            x[k][0] = v; x[k][1] = v ^ 1u; x[k][2] = v ^ 2u; x[k][3] = v ^ 3u;
        }
    }
    if constexpr (WV == 16) {
        GLOBAL u32x4 *d = (GLOBAL u32x4 *)(uint64_t)(dst + c * (STEPS * 256 * 16));
#pragma unroll
        for (int k = 0; k < STEPS; k++) st<u32x4, NTS>(u32x4{x[k][0], x[k][1], x[k][2], x[k][3]}, d + k * 256 + t);
    } else if constexpr (WV == 8) {
        GLOBAL u32x2 *d = (GLOBAL u32x2 *)(uint64_t)(dst + c * (STEPS * 256 * 8));
#pragma unroll
        for (int k = 0; k < STEPS; k++) st<u32x2, NTS>(u32x2{x[k][0] ^ x[k][1], x[k][2] ^ x[k][3]}, d + k * 256 + t);
    } else if constexpr (WV == 4) {
        GLOBAL u32 *d = (GLOBAL u32 *)(uint64_t)(dst + c * (STEPS * 256 * 4));
#pragma unroll
        for (int k = 0; k < STEPS; k++) st<u32, NTS>(x[k][0] ^ x[k][1] ^ x[k][2] ^ x[k][3], d + k * 256 + t);
    } else if constexpr (WV == 2) {
        u32x4 a = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < STEPS; k++) a ^= u32x4{x[k][0], x[k][1], x[k][2], x[k][3]};
        GLOBAL u32x4 *d = (GLOBAL u32x4 *)(uint64_t)(dst + c * (256 * 16));
        st<u32x4, NTS>(a, d + t);
    } else {  // read only: the loads must not be optimised away
        u32 a = 0;
#pragma unroll
        for (int k = 0; k < STEPS; k++) a ^= x[k][0] ^ x[k][1] ^ x[k][2] ^ x[k][3];
        if (a == never) *(GLOBAL u32 *)(uint64_t)dst = a;
    }
}

// piece of work of workgroup id b: see `eighths` in the file header
__device__ __forceinline__ int piece_of(int per_xcd)
{
    return per_xcd > 0 ? (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
}

template <bool NTL, bool LINE, bool NTS>
__global__ __launch_bounds__(256) void k_reduce_pattern(uint8_t *buf, int64_t slot_size, int rows, int row_bytes,
                                                        int rank, int per_xcd)
{
    const int j = piece_of(per_xcd);
    if (j >= rows) return;
    const int t = threadIdx.x;
    const int ndw = (row_bytes >> 2) - 1;
    const int doff = min(4 * t, ndw - 4);  // the last vector of a row is moved back to end with the row
    const int64_t off = (int64_t)j * row_bytes;
    u32x4 w[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int peer = (rank + k) & 7;
        GLOBAL const u32 *pv = (GLOBAL const u32 *)(uint64_t)(buf + peer * slot_size + off) + 1;
        uint64_t addr = (uint64_t)(pv + doff);  // 4-byte aligned 16-byte access
        if (LINE) addr = ((uint64_t)(pv + (doff & ~255)) & ~(uint64_t)127) + 16 * (t & 63);
        GLOBAL const u32x4_a4 *q = (GLOBAL const u32x4_a4 *)addr;
        w[k] = NTL ? __builtin_nontemporal_load(q) : *q;
    }
    u32x4 a = w[0];
#pragma unroll
    for (int k = 1; k < 8; k++) a ^= w[k];
    GLOBAL u32 *orow = (GLOBAL u32 *)(uint64_t)(buf + rank * slot_size + off);
    uint64_t oaddr = (uint64_t)(orow + 1 + doff);
    if (LINE) oaddr = ((uint64_t)(orow + 1 + (doff & ~255)) & ~(uint64_t)127) + 16 * (t & 63);
    if (4 * t < ndw) {
        if (NTS) __builtin_nontemporal_store(a, (GLOBAL u32x4_a4 *)oaddr);
        else *(GLOBAL u32x4_a4 *)oaddr = a;
    }
    if (t == 0) orow[0] = a.x;
}

// Reduce's accesses on a slot that holds two kinds of rows, for a group of WS peers (WS * UNITS
// = 8 loads per lane): rows_b rows of row_bytes_b (more than 1024 and at most 2048 payload
// dwords: one workgroup per row, two vectors per lane and peer in the lower wavefronts, as many
// as the row needs in the upper ones) from byte off_b of every slot, handed out first, then
// rows_a rows of row_bytes_a (at most 512 payload dwords: one wavefront per row, two vectors per
// lane and peer) from byte off_a.  Chunks of 2^chunk_shift consecutive workgroups go to the 8
// XCDs in turn, as the product hands out the work of long tensor lists.
template <int WS, bool NTL, bool NTS>
__global__ __launch_bounds__(256) void k_reduce_pattern_mix(uint8_t *buf, int64_t slot_size, int rank, int rows_a,
                                                            int row_bytes_a, int64_t off_a, int rows_b, int row_bytes_b,
                                                            int64_t off_b, int chunk_shift, int nwg)
{
    constexpr int UNITS = 8 / WS;
    const int i = (int)(blockIdx.x >> 3), x = (int)(blockIdx.x & 7), cs = chunk_shift;
    const int vb = ((((i >> cs) << 3) + x) << cs) + (i & ((1 << cs) - 1));
    if (vb >= nwg) return;
    const int t = threadIdx.x, wave = t >> 6;
    int team, lane, ndw, units = UNITS;
    int64_t off;
    if (vb < rows_b) {
        team = 256; lane = t;
        ndw = (row_bytes_b >> 2) - 1;
        off = off_b + (int64_t)vb * row_bytes_b;
        units = min(UNITS, max(1, (ndw - 256 * wave + 1023) >> 10));
    } else {
        const int j = (vb - rows_b) * 4 + wave;
        if (j >= rows_a) return;
        team = 64; lane = t & 63;
        ndw = (row_bytes_a >> 2) - 1;
        off = off_a + (int64_t)j * row_bytes_a;
    }
    int doff[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; u++) doff[u] = min(4 * (u * team + lane), ndw - 4);
    u32x4 w[WS][UNITS];
#pragma unroll
    for (int k = 0; k < WS; k++) {
        int peer = rank + k;
        if (peer >= WS) peer -= WS;
        GLOBAL const u32 *pv = (GLOBAL const u32 *)(uint64_t)(buf + peer * slot_size + off) + 1;
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            GLOBAL const u32x4_a4 *q = (GLOBAL const u32x4_a4 *)(pv + doff[u < units ? u : 0]);
            w[k][u] = NTL ? __builtin_nontemporal_load(q) : *q;
        }
    }
    GLOBAL u32 *orow = (GLOBAL u32 *)(uint64_t)(buf + rank * slot_size + off);
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        u32x4 a = w[0][u];
#pragma unroll
        for (int k = 1; k < WS; k++) a ^= w[k][u];
        if (u < units && 4 * (u * team + lane) < ndw) {
            if (NTS) __builtin_nontemporal_store(a, (GLOBAL u32x4_a4 *)(orow + 1 + doff[u]));
            else *(GLOBAL u32x4_a4 *)(orow + 1 + doff[u]) = a;
        }
        if (u == 0 && lane == 0) orow[0] = a.x;
    }
}

template <bool NTL, bool NTS>
__global__ __launch_bounds__(256) void k_dequantize_pattern(const uint8_t *packed, uint8_t *tensor, int rows,
                                                            int row_bytes, int per_xcd)
{
    const int r = piece_of(per_xcd) * 4 + (int)(threadIdx.x >> 6);
    if (r >= rows) return;
    const int l = threadIdx.x & 63;
    GLOBAL const u32x2_a4 *pk = (GLOBAL const u32x2_a4 *)(uint64_t)(packed + (int64_t)r * row_bytes + 4);
    GLOBAL u32x4 *tn = (GLOBAL u32x4 *)(uint64_t)(tensor + (int64_t)r * 8192);
    u32x2 w[8];
#pragma unroll
    for (int k = 0; k < 8; k++) w[k] = NTL ? __builtin_nontemporal_load(pk + k * 64 + l) : pk[k * 64 + l];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const u32x4 o = {w[k].x, w[k].y, w[k].x ^ 1u, w[k].y ^ 1u};
        if (NTS) __builtin_nontemporal_store(o, tn + k * 64 + l);
        else tn[k * 64 + l] = o;
    }
}

template <bool NTL, bool STAGED>
__global__ __launch_bounds__(256) void k_quantize_pattern(const uint8_t *tensor, uint8_t *packed, int rows,
                                                          int row_bytes, int per_xcd)
{
    __shared__ __align__(16) uint8_t stage[16640];
    const int r0 = piece_of(per_xcd) * 4;
    if (r0 >= rows) return;  // rows is a multiple of 4
    const int t = threadIdx.x, wave = t >> 6, l = t & 63;
    GLOBAL const u32x4 *in = (GLOBAL const u32x4 *)(uint64_t)(tensor + (int64_t)(r0 + wave) * 8192);
    u32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = NTL ? __builtin_nontemporal_load(in + k * 64 + l) : in[k * 64 + l];
    uint8_t *g0 = packed + (int64_t)r0 * row_bytes;
    if (STAGED) {
        const int mis = (int)((uint64_t)g0 & 127u);
        typedef __attribute__((address_space(3))) uint8_t lds_u8;
        lds_u8 *srow = (lds_u8 *)stage + mis + wave * row_bytes;
        if (l == 0) *(__attribute__((address_space(3))) u32 *)srow = v[0].x;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const u32x2 o = {v[k].x ^ v[k].z, v[k].y ^ v[k].w};
            *(__attribute__((address_space(3))) u32x2_a4 *)(srow + 4 + 8 * (k * 64 + l)) = o;
        }
        __syncthreads();
        const int end = mis + 4 * row_bytes;
        GLOBAL uint8_t *line0 = (GLOBAL uint8_t *)(uint64_t)(g0 - mis);
        for (int c = t; c < (end + 15) >> 4; c += 256) {
            const int lo = 16 * c;
            const u32x4 x = *(const __attribute__((address_space(3))) u32x4 *)((lds_u8 *)stage + lo);
            if (lo >= mis && lo + 16 <= end) {
                __builtin_nontemporal_store(x, (GLOBAL u32x4 *)(line0 + lo));
            } else {
                const u32 w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
                for (int d = 0; d < 4; d++)
                    if (lo + 4 * d >= mis && lo + 4 * d < end) *(GLOBAL u32 *)(line0 + lo + 4 * d) = w[d];
            }
        }
    } else {
        GLOBAL u32 *out = (GLOBAL u32 *)(uint64_t)(g0 + (int64_t)wave * row_bytes);
        if (l == 0) out[0] = v[0].x;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const u32x2 o = {v[k].x ^ v[k].z, v[k].y ^ v[k].w};
            *(GLOBAL u32x2_a4 *)(out + 1 + 2 * (k * 64 + l)) = o;
        }
    }
}

// Bytes that one launch of `kind` reads and writes; units = workgroups of the plain mixes, rows
// of the patterns.
extern "C" int tftq_ceiling_bytes(int kind, int64_t units, int row_bytes, int64_t *read_bytes, int64_t *write_bytes)
{
    static const int rv[7] = {16, 0, 16, 8, 16, 4, 16}, wv[7] = {0, 16, 8, 16, 4, 16, 2};
    if (kind < 0 || kind >= C_KINDS || !read_bytes || !write_bytes) return -1;
    if (kind == C_DEQ) {
        *read_bytes = units * (int64_t)row_bytes;
        *write_bytes = units * 8192;
    } else if (kind == C_QNT) {
        *read_bytes = units * 8192;
        *write_bytes = units * (int64_t)row_bytes;
    } else if (kind == C_RED || kind == C_RED_LINE) {
        *read_bytes = units * (int64_t)row_bytes * 8;
        *write_bytes = units * (int64_t)row_bytes;
    } else if (kind >= C_R2W1_4) {
        *read_bytes = units * 4 * 256 * (int64_t)rv[kind - C_R2W1_4 + C_R2W1];
        *write_bytes = units * 4 * 256 * (int64_t)wv[kind - C_R2W1_4 + C_R2W1];
    } else {
        *read_bytes = units * 8 * 256 * (int64_t)rv[kind];
        *write_bytes = units * 8 * 256 * (int64_t)wv[kind];
    }
    return 0;
}

// One launch on `stream`.  Plain mixes: src and dst hold what tftq_ceiling_bytes says.  RED,
// RED_LINE: dst is the buffer of 8 slots of slot_size bytes, updated in place (RED_LINE: slot_size
// a multiple of 128), src is not used, 20 <= row_bytes <= 4100.  DEQ: src holds the packed rows
// (row_bytes >= 4100 apart), dst the rows of 8192 bytes.  QNT: src holds rows of 8192 bytes, dst
// the packed rows (row_bytes = 4100, units a multiple of 4).  nt_loads / nt_stores pick streaming
// (nontemporal) accesses (RED, RED_LINE: of the codes; the scale dword is a plain store).
// Returns 0, a hipError_t, or -1 for bad arguments.
extern "C" int tftq_ceiling_launch(int kind, const void *src, void *dst, int64_t units, int64_t slot_size,
                                   int row_bytes, int rank, int eighths, int nt_loads, int nt_stores, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    const dim3 block(256);
    const uint8_t *a = (const uint8_t *)src;
    uint8_t *b = (uint8_t *)dst;
    if (units <= 0) return 0;
    if (units > 0x7FFFFFF0) return -1;
    const dim3 grid((unsigned)units);
#define TFTQ_C(RV, WV) TFTQ_CS(RV, WV, 8)
#define TFTQ_CS(RV, WV, STEPS)                                                                             \
    do {                                                                                                   \
        if (nt_loads && nt_stores) hipLaunchKernelGGL((k_stream<RV, WV, true, true, STEPS>), grid, block, 0, s, a, b, units, 0x9E3779B9u);  \
        else if (nt_loads) hipLaunchKernelGGL((k_stream<RV, WV, true, false, STEPS>), grid, block, 0, s, a, b, units, 0x9E3779B9u);          \
        else if (nt_stores) hipLaunchKernelGGL((k_stream<RV, WV, false, true, STEPS>), grid, block, 0, s, a, b, units, 0x9E3779B9u);         \
        else hipLaunchKernelGGL((k_stream<RV, WV, false, false, STEPS>), grid, block, 0, s, a, b, units, 0x9E3779B9u);                       \
    } while (0)
    switch (kind) {
    case C_RO: TFTQ_C(16, 0); break;
    case C_WO: TFTQ_C(0, 16); break;
    case C_R2W1: TFTQ_C(16, 8); break;
    case C_R1W2: TFTQ_C(8, 16); break;
    case C_R4W1: TFTQ_C(16, 4); break;
    case C_R1W4: TFTQ_C(4, 16); break;
    case C_R8W1: TFTQ_C(16, 2); break;
    case C_R2W1_4: TFTQ_CS(16, 8, 4); break;
    case C_R1W2_4: TFTQ_CS(8, 16, 4); break;
    case C_R4W1_4: TFTQ_CS(16, 4, 4); break;
    case C_R1W4_4: TFTQ_CS(4, 16, 4); break;
    case C_RED:
    case C_RED_LINE: {
        if (row_bytes < 20 || row_bytes > 4100 || (row_bytes & 3) || rank < 0 || rank > 7) return -1;
        if (kind == C_RED_LINE && (slot_size & 127)) return -1;
        const int px = eighths ? (int)((units + 7) / 8) : 0;
        const dim3 g(eighths ? (unsigned)(8 * px) : (unsigned)units);
        const int rows = (int)units;
#define TFTQ_RED(LINE)                                                                                              \
    do {                                                                                                            \
        if (nt_loads && nt_stores) hipLaunchKernelGGL((k_reduce_pattern<true, LINE, true>), g, block, 0, s, b, slot_size, rows, row_bytes, rank, px);        \
        else if (nt_loads) hipLaunchKernelGGL((k_reduce_pattern<true, LINE, false>), g, block, 0, s, b, slot_size, rows, row_bytes, rank, px);              \
        else if (nt_stores) hipLaunchKernelGGL((k_reduce_pattern<false, LINE, true>), g, block, 0, s, b, slot_size, rows, row_bytes, rank, px);             \
        else hipLaunchKernelGGL((k_reduce_pattern<false, LINE, false>), g, block, 0, s, b, slot_size, rows, row_bytes, rank, px);                           \
    } while (0)
        if (kind == C_RED) TFTQ_RED(false);
        else TFTQ_RED(true);
#undef TFTQ_RED
        break;
    }
    case C_DEQ: {
        if (row_bytes < 4100 || (row_bytes & 3)) return -1;
        const int wgs = (int)((units + 3) / 4);
        const int px = eighths ? (wgs + 7) / 8 : 0;
        const dim3 g(eighths ? (unsigned)(8 * px) : (unsigned)wgs);
        const int rows = (int)units;
        if (nt_loads && nt_stores) hipLaunchKernelGGL((k_dequantize_pattern<true, true>), g, block, 0, s, a, b, rows, row_bytes, px);
        else if (nt_loads) hipLaunchKernelGGL((k_dequantize_pattern<true, false>), g, block, 0, s, a, b, rows, row_bytes, px);
        else if (nt_stores) hipLaunchKernelGGL((k_dequantize_pattern<false, true>), g, block, 0, s, a, b, rows, row_bytes, px);
        else hipLaunchKernelGGL((k_dequantize_pattern<false, false>), g, block, 0, s, a, b, rows, row_bytes, px);
        break;
    }
    case C_QNT: {
        if (row_bytes != 4100 || (units & 3)) return -1;
        const int wgs = (int)(units / 4);
        const int px = eighths ? (wgs + 7) / 8 : 0;
        const dim3 g(eighths ? (unsigned)(8 * px) : (unsigned)wgs);
        const int rows = (int)units;
        if (nt_loads && nt_stores) hipLaunchKernelGGL((k_quantize_pattern<true, true>), g, block, 0, s, a, b, rows, row_bytes, px);
        else if (nt_loads) hipLaunchKernelGGL((k_quantize_pattern<true, false>), g, block, 0, s, a, b, rows, row_bytes, px);
        else if (nt_stores) hipLaunchKernelGGL((k_quantize_pattern<false, true>), g, block, 0, s, a, b, rows, row_bytes, px);
        else hipLaunchKernelGGL((k_quantize_pattern<false, false>), g, block, 0, s, a, b, rows, row_bytes, px);
        break;
    }
    default: return -1;
    }
#undef TFTQ_C
    return (int)hipGetLastError();
}

// One launch of k_reduce_pattern_mix on `stream` (see there): buf holds ws slots of slot_size
// bytes and is updated in place; ws is 4 or 8; nt_loads / nt_stores pick streaming accesses for
// the codes (the scale dword is always a plain store).  Reads ws times, writes once, the
// rows_a * row_bytes_a + rows_b * row_bytes_b bytes of a slot's rows.
extern "C" int tftq_ceiling_reduce_mix(void *buf, int64_t slot_size, int ws, int rank, int rows_a, int row_bytes_a,
                                       int64_t off_a, int rows_b, int row_bytes_b, int64_t off_b, int chunk_shift,
                                       int nt_loads, int nt_stores, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    if (!buf || (ws != 4 && ws != 8) || rank < 0 || rank >= ws || rows_a < 0 || rows_b < 0) return -1;
    if ((row_bytes_a & 3) || (row_bytes_b & 3) || row_bytes_a < 20 || row_bytes_a > 2052) return -1;
    if (rows_b > 0 && (row_bytes_b <= 4100 || row_bytes_b > 8196)) return -1;
    if (chunk_shift < 0 || chunk_shift > 16) return -1;
    const int nwg = rows_b + (rows_a + 3) / 4;
    if (nwg == 0) return 0;
    const int chunk = 1 << chunk_shift;
    const int chunks = (nwg + chunk - 1) / chunk;
    const int per_xcd = (chunks + 7) / 8 * chunk;
    const dim3 grid((unsigned)(8 * per_xcd)), block(256);
    uint8_t *b = (uint8_t *)buf;
#define TFTQ_MIX(WS, NTL, NTS)                                                                                        \
    hipLaunchKernelGGL((k_reduce_pattern_mix<WS, NTL, NTS>), grid, block, 0, s, b, slot_size, rank, rows_a, row_bytes_a, \
                       off_a, rows_b, row_bytes_b, off_b, chunk_shift, nwg)
#define TFTQ_MIX_W(WS)                                                                     \
    do {                                                                                   \
        if (nt_loads && nt_stores) TFTQ_MIX(WS, true, true);                               \
        else if (nt_loads) TFTQ_MIX(WS, true, false);                                      \
        else if (nt_stores) TFTQ_MIX(WS, false, true);                                     \
        else TFTQ_MIX(WS, false, false);                                                   \
    } while (0)
    if (ws == 4) TFTQ_MIX_W(4);
    else TFTQ_MIX_W(8);
#undef TFTQ_MIX_W
#undef TFTQ_MIX
    return (int)hipGetLastError();
}
