// HIP kernels for gfx950 (MI355X) and the compute entry points of the C ABI.
//
// Three kernels, one launch per stage:
//   k_quantize<T>    fused_quantize_into_fp8   (torchft/quantization.py:53-162)
//   k_reduce         fused_reduce_fp8          (:261-428)
//   k_dequantize<T>  fused_dequantize_from_fp8 (:165-258)
//
// Design (none of it follows the reference's launch shape):
//   * a row is owned by a "team" of 1, 8, 64 or 256 lanes chosen from the row
//     length; the team loads the row once with 16-byte loads, keeps it in
//     registers, reduces |x| with DPP inside the wavefront (LDS across the four
//     wavefronts of a 256-lane team) and converts from registers with the
//     packed fp8 converts of gfx950.  Every stage reads HBM once.
//   * all tensors of a call are covered by one launch: a workgroup finds its
//     tensor in a table of 64-byte descriptors (in the kernel arguments for
//     short lists) and branches on the team size stored there.
//   * workgroup ids are remapped so that each of the 8 XCDs works on one
//     contiguous range of rows (neighbouring packed rows share cache lines).
//   * division by a row scale is exact IEEE division, computed as
//     fma(f, r, f * r_lo) with r = RN(1/s) and r_lo = RN(fma(-s, r, 1) / s).
//     For the 253 finite e4m3 values f and every binary32 s with exponent in
//     [-64, 64] this equals RN(f / s) bit for bit (checked exhaustively by
//     tests/test_exact_division.py); other scales take the plain divide.
//
// Build flags that matter: -ffp-contract=off (the arithmetic contract is
// separate IEEE multiply / divide / add), packed fp32 ops disabled.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "../../include/tftq.h"
#include "tftq_internal.h"

typedef uint32_t u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x2 u32x2_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));  // tensor rows: aligned to the element only
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct bf16_tag {};
struct f16_tag {};

#define DEV __device__ __forceinline__
// Streaming accesses for data that is touched once per kernel (measured on
// MI355X: +10 % read bandwidth over plain loads).
#define LOAD_STREAM(ptr) __builtin_nontemporal_load(ptr)
#define STORE_STREAM(val, ptr) __builtin_nontemporal_store((val), (ptr))
#define GLOBAL __attribute__((address_space(1)))

// Tensor addresses arrive as integers; tell the compiler they are global
// memory so that it emits global_* rather than flat_* accesses.
template <typename P>
DEV GLOBAL P *as_global(uint64_t addr)
{
    return (GLOBAL P *)addr;
}
template <typename P>
DEV GLOBAL P *as_global(const void *ptr)
{
    return (GLOBAL P *)(uint64_t)ptr;
}

DEV float as_f(u32 u) { return __uint_as_float(u); }
DEV u32 as_u(float f) { return __float_as_uint(f); }

// ---------------------------------------------------------------------------
// wavefront / team reductions
// ---------------------------------------------------------------------------
template <int CTRL>
DEV float dpp_mov(float v)
{
    const int x = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false));
}

DEV float bcast_lane(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// v of lane k of the caller's team (k uniform).  Teams of whole wavefronts hold
// the same values in every wavefront and read lane k; smaller teams go through
// the LDS crossbar.
template <int TEAM>
DEV float team_bcast(float v, int k)
{
    if constexpr (TEAM >= 64) {
        return bcast_lane(v, k);
    } else {
        const int base = (int)(threadIdx.x & 63u) & ~(TEAM - 1);
        return __int_as_float(__builtin_amdgcn_ds_bpermute((base + k) << 2, __float_as_int(v)));
    }
}

// max over the TEAM lanes that share a row; every lane of the team gets it.
// lds: 4 floats per workgroup, used by 256-lane teams only.
template <int TEAM>
DEV float team_max(float v, float *lds)
{
    if (TEAM >= 8) {
        v = fmaxf(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
        v = fmaxf(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
        v = fmaxf(v, dpp_mov<0x141>(v));  // row_half_mirror
    }
    if (TEAM >= 16) v = fmaxf(v, dpp_mov<0x140>(v));  // row_mirror: all 16 lanes of a row agree
    if (TEAM >= 32) {
        const float a = bcast_lane(v, 0), b = bcast_lane(v, 16);
        const float c = bcast_lane(v, 32), d = bcast_lane(v, 48);
        if (TEAM == 32) v = (threadIdx.x & 32) ? fmaxf(c, d) : fmaxf(a, b);
        else v = fmaxf(fmaxf(a, b), fmaxf(c, d));
    }
    if (TEAM == 256) {
        const int wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) lds[wave] = v;
        __syncthreads();
        v = fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
        __syncthreads();
    }
    return v;
}

// ---------------------------------------------------------------------------
// scalar helpers of the arithmetic contract
// ---------------------------------------------------------------------------
// _kernel_calculate_scale (quantization.py:44-50)
DEV float calc_scale(float row_max)
{
    const float s = 448.0f / row_max;
    return s == __builtin_inff() ? 1.0f : s;
}

// Exact f / s for e4m3 values f (see the file header).
struct DivCoef {
    float s, r, r_lo;
    bool fast;
};

// positive, exponent in [-64, 64]
DEV bool scale_is_fast(float s) { return (as_u(s) - (63u << 23)) < (129u << 23); }

DEV DivCoef make_div(float s)
{
    DivCoef c;
    c.s = s;
    c.r = 1.0f / s;
    c.r_lo = __builtin_fmaf(-s, c.r, 1.0f) / s;
    c.fast = scale_is_fast(s);
    return c;
}

DEV float div_fast(float f, float r, float r_lo) { return __builtin_fmaf(f, r, f * r_lo); }

// Same, with the sign of a zero numerator kept (-0 / s = -0 for s > 0; the fma
// form gives +0).  The sum in reduce cannot tell the two zeros apart, the
// stored result of dequantize can.
DEV float div_fast_signed(float f, float r, float r_lo)
{
    return __builtin_copysignf(div_fast(f, r, r_lo), f);
}

// four e4m3 codes -> four floats
DEV void unpack_fp8x4(u32 w, float (&f)[4])
{
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    f[0] = lo.x; f[1] = lo.y; f[2] = hi.x; f[3] = hi.y;
}

// four floats -> four e4m3 codes (round to nearest even, no saturation)
DEV u32 pack_fp8x4(float a, float b, float c, float d)
{
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (u32)w;
}

// ---------------------------------------------------------------------------
// element types
// ---------------------------------------------------------------------------
template <typename T> struct Elem;

template <> struct Elem<float> {
    static constexpr int ESZ = 4;
    static constexpr int EPV = 4;  // elements per 16-byte vector
    DEV static void unpack(const u32x4 v, float (&f)[4])
    {
        f[0] = as_f(v.x); f[1] = as_f(v.y); f[2] = as_f(v.z); f[3] = as_f(v.w);
    }
    DEV static u32x4 pack(const float (&f)[4])
    {
        u32x4 v = {as_u(f[0]), as_u(f[1]), as_u(f[2]), as_u(f[3])};
        return v;
    }
    DEV static float load(uint64_t base, int64_t idx) { return as_global<const float>(base)[idx]; }
    DEV static void store(uint64_t base, int64_t idx, float v) { as_global<float>(base)[idx] = v; }
};

template <> struct Elem<bf16_tag> {
    static constexpr int ESZ = 2;
    static constexpr int EPV = 8;
    DEV static void unpack(const u32x4 v, float (&f)[8])
    {
        f[0] = as_f(v.x << 16); f[1] = as_f(v.x & 0xFFFF0000u);
        f[2] = as_f(v.y << 16); f[3] = as_f(v.y & 0xFFFF0000u);
        f[4] = as_f(v.z << 16); f[5] = as_f(v.z & 0xFFFF0000u);
        f[6] = as_f(v.w << 16); f[7] = as_f(v.w & 0xFFFF0000u);
    }
    DEV static u32 pack2(float a, float b)
    {
        const f32x2 p = {a, b};
        const bf16x2 h = __builtin_convertvector(p, bf16x2);  // round to nearest even
        return __builtin_bit_cast(u32, h);
    }
    DEV static u32x4 pack(const float (&f)[8])
    {
        u32x4 v = {pack2(f[0], f[1]), pack2(f[2], f[3]), pack2(f[4], f[5]), pack2(f[6], f[7])};
        return v;
    }
    DEV static float load(uint64_t base, int64_t idx)
    {
        return as_f((u32)as_global<const uint16_t>(base)[idx] << 16);
    }
    DEV static void store(uint64_t base, int64_t idx, float v)
    {
        as_global<uint16_t>(base)[idx] = (uint16_t)(pack2(v, 0.0f) & 0xFFFFu);
    }
};

template <> struct Elem<f16_tag> {
    static constexpr int ESZ = 2;
    static constexpr int EPV = 8;
    DEV static void unpack2(u32 w, float &a, float &b)
    {
        const f16x2 h = __builtin_bit_cast(f16x2, w);
        a = (float)h.x;
        b = (float)h.y;
    }
    DEV static void unpack(const u32x4 v, float (&f)[8])
    {
        unpack2(v.x, f[0], f[1]); unpack2(v.y, f[2], f[3]);
        unpack2(v.z, f[4], f[5]); unpack2(v.w, f[6], f[7]);
    }
    // The value is first rounded to binary32, then to binary16.  Hide the
    // producer from the compiler: it would otherwise fuse fma + convert into
    // v_fma_mixlo_f16, which rounds once and differs in the last bit.
    DEV static float opaque(float x)
    {
        asm("" : "+v"(x));
        return x;
    }
    DEV static u32 pack2(float a, float b)
    {
        f16x2 h;
        h.x = (_Float16)opaque(a);  // round to nearest even
        h.y = (_Float16)opaque(b);
        return __builtin_bit_cast(u32, h);
    }
    DEV static u32x4 pack(const float (&f)[8])
    {
        u32x4 v = {pack2(f[0], f[1]), pack2(f[2], f[3]), pack2(f[4], f[5]), pack2(f[6], f[7])};
        return v;
    }
    DEV static float load(uint64_t base, int64_t idx)
    {
        return (float)as_global<const _Float16>(base)[idx];
    }
    DEV static void store(uint64_t base, int64_t idx, float v)
    {
        as_global<_Float16>(base)[idx] = (_Float16)opaque(v);
    }
};

// ---------------------------------------------------------------------------
// workgroup -> (segment, first row)
// ---------------------------------------------------------------------------
// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2.  Workgroup id b is the (b >> 3)-th piece of work of XCD b & 7.
//
// Inline table (at most 16 segments): XCD x takes the x-th contiguous eighth of
// every segment's workgroups and walks the segments in the stage's work order
// (reduce: heaviest workgroups first, so that every XCD sees the same mix of
// row lengths and the last workgroups to finish are light).
// Device table (longer lists): workgroup numbers follow the segments in the
// stage's work order, chunks of consecutive numbers go to the XCDs in turn, and
// a bucket map plus a short binary search lead from the number to the segment.
// Ids past the end of their XCD's work return false.
//
// The kernel arguments are (KParams, InlineTable).  Indexing those by-value
// structs with a run-time index would make the compiler copy them to private
// memory; reading the kernel-argument segment through a constant-address-space
// pointer keeps the accesses scalar loads.
#define CONSTANT __attribute__((address_space(4)))
constexpr size_t KARG_TABLE_OFF = (sizeof(KParams) + alignof(InlineTable) - 1) / alignof(InlineTable) * alignof(InlineTable);

DEV const CONSTANT Seg *karg_table()
{
    return (const CONSTANT Seg *)((const CONSTANT char *)__builtin_amdgcn_kernarg_segment_ptr() + KARG_TABLE_OFF);
}

template <bool INLINE, int STAGE>
DEV bool locate(const KParams &p, const InlineTable &inl, Seg &s, int &vb)
{
    const int x = (int)(blockIdx.x & 7);
    const int i = (int)(blockIdx.x >> 3);
    if (INLINE) {
        // One round of scalar loads fetches this XCD's three table rows; the position
        // is then found in registers, and only the segment descriptor needs a second round.
        const CONSTANT char *karg = (const CONSTANT char *)__builtin_amdgcn_kernarg_segment_ptr();
        const CONSTANT int32_t *d = (const CONSTANT int32_t *)(karg + offsetof(KParams, dealt)) + x * TFTQ_N_INLINE;
        typedef int32_t Row __attribute__((ext_vector_type(TFTQ_N_INLINE)));  // one 64-byte scalar load
        const Row cum_end = *(const CONSTANT Row *)(d + offsetof(Dealt, cum_end) / 4);
        const Row base = *(const CONSTANT Row *)(d + offsetof(Dealt, base) / 4);
        const Row seg = *(const CONSTANT Row *)(d + offsetof(Dealt, seg) / 4);
        Row cum_end_ = cum_end, base_ = base, seg_ = seg;
        // all scalar loads of this round, and the common parameters, are issued before the first wait
        asm volatile("" : "+s"(cum_end_), "+s"(base_), "+s"(seg_) : "s"(p.packed), "s"(p.slot_size), "s"(p.ws), "s"(p.rank));
        int b = base_[0], sg = seg_[0];
#pragma unroll
        for (int j = 1; j < TFTQ_N_INLINE; j++) {
            const bool past = i >= cum_end_[j - 1];  // cum_end is non-decreasing: the last hit wins
            b = past ? base_[j] : b;
            sg = past ? seg_[j] : sg;
        }
        if (sg < 0 || i >= cum_end_[TFTQ_N_INLINE - 1]) return false;
        vb = b + i;
        const CONSTANT u32x4 *src = (const CONSTANT u32x4 *)(karg_table() + sg);
        const u32x4 v[4] = {src[0], src[1], src[2], src[3]};
        __builtin_memcpy(&s, v, sizeof(Seg));
        return true;
    } else {
        // everything the first steps need from the kernel arguments in one round of scalar loads
        asm volatile("" ::"s"(p.table), "s"(p.map_off), "s"(p.sorted_off), "s"(p.map_shift), "s"(p.chunk_shift), "s"(p.nwg),
                     "s"(p.packed), "s"(p.slot_size), "s"(p.ws), "s"(p.rank));
        // chunks of 2^chunk_shift consecutive workgroups go to the XCDs in turn
        const int cs = p.chunk_shift;
        vb = ((((i >> cs) << 3) + x) << cs) + (i & ((1 << cs) - 1));
        if (vb >= p.nwg) return false;
        const uint64_t tab = (uint64_t)p.table;
        typedef int32_t MapPair __attribute__((ext_vector_type(4), aligned(8)));
        const MapPair m = *(const CONSTANT MapPair *)(tab + (uint64_t)p.map_off +
                                                      (uint64_t)(vb >> p.map_shift) * sizeof(MapEnt));
        int lo = m.x, sg = m.y, hi = m.z;
        if (lo != hi) {  // last position whose first workgroup is <= vb
            const CONSTANT SortEnt *sorted = (const CONSTANT SortEnt *)(tab + (uint64_t)p.sorted_off);
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (sorted[mid].begin <= vb) lo = mid; else hi = mid - 1;
            }
            sg = sorted[lo].seg;
        }
        const CONSTANT u32x4 *src = (const CONSTANT u32x4 *)(tab + (uint64_t)sg * sizeof(Seg));
        const u32x4 v[4] = {src[0], src[1], src[2], src[3]};
        __builtin_memcpy(&s, v, sizeof(Seg));
        return true;
    }
}

DEV int64_t row_addr(const Seg &s, int64_t slot_size, int row)
{
    const int slot = row / s.slice_rows;
    const int j = row - slot * s.slice_rows;
    return (int64_t)slot * slot_size + s.slot_off + (int64_t)j * s.row_bytes;
}

// ---------------------------------------------------------------------------
// quantize
// ---------------------------------------------------------------------------
constexpr int QV = 8;  // 16-byte vectors a lane keeps in registers

template <typename T>
DEV float vec_absmax(const u32x4 v)
{
    float f[Elem<T>::EPV];
    Elem<T>::unpack(v, f);
    float a = 0.0f;
#pragma unroll
    for (int e = 0; e < Elem<T>::EPV; e++) a = fmaxf(a, __builtin_fabsf(f[e]));
    return a;
}

template <typename T>
DEV void vec_quant_store(const u32x4 v, float s, GLOBAL u32 *payload, int idx)
{
    float f[Elem<T>::EPV];
    Elem<T>::unpack(v, f);
    if constexpr (Elem<T>::EPV == 4) {
        payload[idx] = pack_fp8x4(f[0] * s, f[1] * s, f[2] * s, f[3] * s);
    } else {
        u32x2 o;
        o.x = pack_fp8x4(f[0] * s, f[1] * s, f[2] * s, f[3] * s);
        o.y = pack_fp8x4(f[4] * s, f[5] * s, f[6] * s, f[7] * s);
        *(GLOBAL u32x2_a4 *)(payload + 2 * idx) = o;  // plain store: rows start 4 bytes off a line, L2 merges
    }
}

// Contiguous, 16-byte aligned rows of at most TEAM * KMAX vectors.  The KMAX
// loads of a lane are issued back to back without a branch in between: lanes
// past the end of the row re-read its last vector (a duplicate cannot change
// the maximum) and simply do not store.
template <typename T, int TEAM, int KMAX>
DEV void quantize_vec_k(const Seg &s, const KParams &p, int row, int lane, float *lds)
{
    const bool active = row < s.slice_rows * p.ws;
    GLOBAL u32 *out = as_global<u32>(p.packed + (active ? row_addr(s, p.slot_size, row) : 0));
    if (active && row >= s.m) {
        // padding row: the reference leaves it zero (:93-95 on a zero-filled buffer)
        for (int d = lane; d < (s.row_bytes >> 2); d += TEAM) out[d] = 0;
    }
    if (!active || row >= s.m) return;  // a team leaves whole: its lanes share the row

    constexpr int EPV = Elem<T>::EPV;
    const int nvec = s.n / EPV;
    const int tail = s.n - nvec * EPV;  // elements after the last whole vector (rare)
    const int64_t r0 = (int64_t)row * s.row_stride;
    GLOBAL const u32x4_a2 *in = as_global<const u32x4_a2>(s.ptr + r0 * Elem<T>::ESZ);
    u32x4 v[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; k++) v[k] = LOAD_STREAM(in + min(k * TEAM + lane, nvec - 1));
    float t[EPV - 1];
    if (tail) {  // every lane reads the few tail elements; lane 0 will store their codes
#pragma unroll
        for (int e = 0; e < EPV - 1; e++) t[e] = Elem<T>::load(s.ptr, r0 + nvec * EPV + min(e, tail - 1));
    }
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < KMAX; k++) amax = fmaxf(amax, vec_absmax<T>(v[k]));
    if (tail) {
#pragma unroll
        for (int e = 0; e < EPV - 1; e++) amax = fmaxf(amax, __builtin_fabsf(t[e]));
    }
    amax = team_max<TEAM>(amax, lds);
    const float sc = calc_scale(amax);
    if (lane == 0) out[0] = as_u(sc);
    // The elements are unpacked again from the raw vectors: keeping the floats of the
    // maximum search alive until here would double the registers of 16-bit inputs.
#pragma unroll
    for (int k = 0; k < KMAX; k++) asm volatile("" : "+v"(v[k].x), "+v"(v[k].y), "+v"(v[k].z), "+v"(v[k].w));
#pragma unroll
    for (int k = 0; k < KMAX; k++) {
        const int idx = k * TEAM + lane;
        if (idx < nvec) vec_quant_store<T>(v[k], sc, out + 1, idx);
    }
    if (tail && lane == 0) {
        float y[8];
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = (e < EPV - 1 && e < tail) ? t[e < EPV - 1 ? e : 0] * sc : 0.0f;
        GLOBAL u32 *tw = out + 1 + nvec * (EPV / 4);
        u32 w0 = pack_fp8x4(y[0], y[1], y[2], y[3]);
        if (tail < 4) w0 &= (1u << (8 * tail)) - 1u;  // padding bytes are zero whatever 0 * sc gave
        tw[0] = w0;
        if (EPV == 8 && tail > 4) {
            u32 w1 = pack_fp8x4(y[4], y[5], y[6], y[7]);
            if (tail < 8) w1 &= (1u << (8 * (tail - 4))) - 1u;
            tw[1] = w1;
        }
    }
}

// Rows of more than 32 KB: too long for the registers of a workgroup.  Two
// passes with 16-byte loads; the second one finds the row in the caches.
template <typename T>
DEV void quantize_vec_long(const Seg &s, const KParams &p, int row, int tid, float *lds)
{
    const bool active = row < s.slice_rows * p.ws;
    if (!active) return;
    GLOBAL u32 *out = as_global<u32>(p.packed + row_addr(s, p.slot_size, row));
    if (row >= s.m) {
        for (int d = tid; d < (s.row_bytes >> 2); d += TFTQ_WG) out[d] = 0;
        return;
    }
    constexpr int EPV = Elem<T>::EPV;
    const int nvec = s.n / EPV;
    const int64_t r0 = (int64_t)row * s.row_stride;
    GLOBAL const u32x4_a2 *in = as_global<const u32x4_a2>(s.ptr + r0 * Elem<T>::ESZ);
    float amax = 0.0f;
    for (int c = nvec * EPV + tid; c < s.n; c += TFTQ_WG) amax = fmaxf(amax, __builtin_fabsf(Elem<T>::load(s.ptr, r0 + c)));
#pragma nounroll
    for (int base = 0; base < nvec; base += 4 * TFTQ_WG) {
        u32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = in[min(base + k * TFTQ_WG + tid, nvec - 1)];
#pragma unroll
        for (int k = 0; k < 4; k++) amax = fmaxf(amax, vec_absmax<T>(v[k]));
    }
    amax = team_max<256>(amax, lds);
    const float sc = calc_scale(amax);
    if (tid == 0) out[0] = as_u(sc);
#pragma nounroll
    for (int base = 0; base < nvec; base += 4 * TFTQ_WG) {
        u32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = LOAD_STREAM(in + min(base + k * TFTQ_WG + tid, nvec - 1));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int idx = base + k * TFTQ_WG + tid;
            if (idx < nvec) vec_quant_store<T>(v[k], sc, out + 1, idx);
        }
    }
    // tail: at most EPV - 1 elements after the last whole vector, byte stores plus zero padding
    if (tid == 0) {
        const int c0 = nvec * EPV;
        GLOBAL uint8_t *ob = (GLOBAL uint8_t *)(out + 1);
        for (int c = c0; c < ((s.n + 3) & ~3); c++) {
            const float x = c < s.n ? Elem<T>::load(s.ptr, r0 + c) : 0.0f;
            ob[c] = c < s.n ? (uint8_t)(pack_fp8x4(x * sc, 0.0f, 0.0f, 0.0f) & 0xFFu) : (uint8_t)0;
        }
    }
}

template <typename T, int TEAM, bool WIDE>
DEV void quantize_vec(const Seg &s, const KParams &p, int row, int lane, float *lds)
{
    // same branch for the whole workgroup
    const int nvec = s.n / Elem<T>::EPV;
    if (nvec <= (QV / 2) * TEAM) quantize_vec_k<T, TEAM, QV / 2>(s, p, row, lane, lds);
    else if (TEAM < 256 || nvec <= TFTQ_Q_VECS) quantize_vec_k<T, TEAM, QV>(s, p, row, lane, lds);
    else if (WIDE && nvec <= TFTQ_Q_VECS_WIDE) quantize_vec_k<T, TEAM, 2 * QV>(s, p, row, lane, lds);
    else quantize_vec_long<T>(s, p, row, lane, lds);
}

// Any strides, any alignment, any n: element loads, two passes over the row
// (the second one is served by the caches).
template <typename T, int TEAM>
DEV void quantize_gen(const Seg &s, const KParams &p, int row, int lane)
{
    const bool active = row < s.slice_rows * p.ws;
    if (!active) return;
    GLOBAL u32 *out = as_global<u32>(p.packed + row_addr(s, p.slot_size, row));
    const int ndw = (s.row_bytes >> 2) - 1;
    if (row >= s.m) {
        for (int d = lane; d <= ndw; d += TEAM) out[d] = 0;
        return;
    }
    const uint64_t base = s.ptr;
    const int64_t r0 = (int64_t)row * s.row_stride;
    float amax = 0.0f;
    for (int c = lane; c < s.n; c += TEAM)
        amax = fmaxf(amax, __builtin_fabsf(Elem<T>::load(base, r0 + (int64_t)c * s.col_stride)));
    amax = team_max<TEAM>(amax, nullptr);
    const float sc = calc_scale(amax);
    if (lane == 0) out[0] = as_u(sc);
    for (int d = lane; d < ndw; d += TEAM) {
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int c = 4 * d + e;
            const float x = c < s.n ? Elem<T>::load(base, r0 + (int64_t)c * s.col_stride) : 0.0f;
            y[e] = x * sc;
        }
        u32 w = pack_fp8x4(y[0], y[1], y[2], y[3]);
        const int tail = s.n - 4 * d;  // codes of this dword that belong to the row
        if (tail < 4) w &= (1u << (8 * tail)) - 1u;  // zero padding, whatever 0 * sc gave
        out[1 + d] = w;
    }
}

// Rows of one column (1-D tensors, quantization.py:487-488): a row is its own
// maximum, so the code is +-448 (or 0) and all information is in the scale.
// Four rows per lane, interleaved so that every load and every 8-byte
// [scale, code] store of a wavefront is contiguous.
template <typename T>
DEV void quantize_col1(const Seg &s, const KParams &p, int row0, int tid)
{
    const int m_pad = s.slice_rows * p.ws;
    float x[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int row = min(row0 + k * TFTQ_WG + tid, s.m - 1);
        x[k] = s.m > 0 ? Elem<T>::load(s.ptr, (int64_t)row * s.row_stride) : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int row = row0 + k * TFTQ_WG + tid;
        if (row < m_pad) {
            u32x2 o = {0u, 0u};  // padding rows stay zero
            if (row < s.m) {
                const float sc = calc_scale(__builtin_fabsf(x[k]));
                o.x = as_u(sc);
                o.y = pack_fp8x4(x[k] * sc, 0.0f, 0.0f, 0.0f) & 0xFFu;
            }
            *(GLOBAL u32x2_a4 *)as_global<u32>(p.packed + row_addr(s, p.slot_size, row)) = o;
        }
    }
}

// Short contiguous rows of whole 16-byte vectors (K_VECS; the shape is
// tftq_small_shape): 1 to 8 lanes per row, and every lane works on several rows
// so that it has 8 loads in flight.  Row slot r of team t is row
// row0 + r * teams + t: for a given r the teams of a wavefront read
// consecutive rows, i.e. consecutive memory.
struct SmallShape {
    int lt, lc, team, teams, nrow, t, l;
};
DEV SmallShape small_shape(int nvec, int tid)
{
    SmallShape h;
    tftq_small_shape(nvec, &h.lt, &h.lc);
    h.team = 1 << h.lt;
    h.teams = TFTQ_WG >> h.lt;
    h.nrow = 8 >> h.lc;
    h.t = tid >> h.lt;
    h.l = tid & (h.team - 1);
    return h;
}

// row -> byte offset of the packed row, with the slot found by one multiply
// (inv = 1.0f / slice_rows; the estimate is off by at most one)
DEV int64_t row_addr_fast(const Seg &s, int64_t slot_size, int row, float inv)
{
    int slot = (int)((float)row * inv);
    int j = row - slot * s.slice_rows;
    if (j < 0) { --slot; j += s.slice_rows; }
    if (j >= s.slice_rows) { ++slot; j -= s.slice_rows; }
    return (int64_t)slot * slot_size + s.slot_off + (int64_t)j * s.row_bytes;
}

template <typename T, int LC>
DEV void quantize_small_c(const Seg &s, const KParams &p, int blk, int tid, const SmallShape &h)
{
    constexpr int EPV = Elem<T>::EPV;
    constexpr int C = 1 << LC, ROWS = 8 >> LC;  // vectors per lane and row, rows per lane
    const int nvec = s.n / EPV;
    const int row0 = blk * (h.teams * ROWS);
    const int m_pad = s.slice_rows * p.ws;
    const float inv = 1.0f / (float)s.slice_rows;

    u32x4 v[ROWS][C];
    int row[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        row[r] = row0 + r * h.teams + h.t;
        const int64_t e0 = (int64_t)min(row[r], s.m - 1) * s.row_stride;  // s.m >= 1: there are rows
        GLOBAL const u32x4_a2 *in = as_global<const u32x4_a2>(s.ptr + e0 * Elem<T>::ESZ);
#pragma unroll
        for (int k = 0; k < C; k++) v[r][k] = LOAD_STREAM(in + min(k * h.team + h.l, nvec - 1));
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < C; k++) a = fmaxf(a, vec_absmax<T>(v[r][k]));
        if (h.lt >= 1) a = fmaxf(a, dpp_mov<0xB1>(a));   // quad_perm [1,0,3,2]
        if (h.lt >= 2) a = fmaxf(a, dpp_mov<0x4E>(a));   // quad_perm [2,3,0,1]
        if (h.lt >= 3) a = fmaxf(a, dpp_mov<0x141>(a));  // row_half_mirror
        if (row[r] >= m_pad) continue;
        GLOBAL u32 *out = as_global<u32>(p.packed + row_addr_fast(s, p.slot_size, row[r], inv));
        if (row[r] >= s.m) {
            // padding row: the reference leaves it zero (:93-95 on a zero-filled buffer)
            for (int d = h.l; d < (s.row_bytes >> 2); d += h.team) out[d] = 0;
            continue;
        }
        const float sc = calc_scale(a);
        if (h.l == 0) out[0] = as_u(sc);
#pragma unroll
        for (int k = 0; k < C; k++)
            if (k * h.team + h.l < nvec) vec_quant_store<T>(v[r][k], sc, out + 1, k * h.team + h.l);
    }
}

template <typename T>
DEV void quantize_small(const Seg &s, const KParams &p, int blk, int tid)
{
    const SmallShape h = small_shape(s.n / Elem<T>::EPV, tid);
    if (h.lc == 0) quantize_small_c<T, 0>(s, p, blk, tid, h);
    else if (h.lc == 1) quantize_small_c<T, 1>(s, p, blk, tid, h);
    else quantize_small_c<T, 2>(s, p, blk, tid, h);
}

template <typename T, bool INLINE, bool WIDE>
__global__ __launch_bounds__(TFTQ_WG) void k_quantize(const KParams p, const InlineTable inl)
{
    __shared__ float lds[4];
    Seg s;
    int vb;
    if (!locate<INLINE, ST_Q>(p, inl, s, vb)) return;
    const int blk = vb - s.wg_begin[ST_Q];
    const int tid = threadIdx.x;
    switch (s.kind[ST_Q]) {
    case K_VEC256: quantize_vec<T, 256, WIDE>(s, p, blk, tid, lds); break;
    case K_VEC64:
        quantize_vec<T, 64, false>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63, lds);
        break;
    case K_VEC32: quantize_vec<T, 32, false>(s, p, blk * 8 + (tid >> 5), tid & 31, lds); break;
    case K_VEC16: quantize_vec<T, 16, false>(s, p, blk * 16 + (tid >> 4), tid & 15, lds); break;
    case K_VEC8: quantize_vec<T, 8, false>(s, p, blk * 32 + (tid >> 3), tid & 7, lds); break;
    case K_GEN64:
        quantize_gen<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_GEN8: quantize_gen<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN1: quantize_gen<T, 1>(s, p, blk * 256 + tid, 0); break;
    case K_COL1: quantize_col1<T>(s, p, blk * 4 * TFTQ_WG, tid); break;
    case K_VECS: quantize_small<T>(s, p, blk, tid); break;
    default: break;
    }
}

// ---------------------------------------------------------------------------
// dequantize
// ---------------------------------------------------------------------------
// Streaming (nontemporal) stores pay off only when the pieces a store instruction
// writes are whole 64-byte blocks: partial blocks written that way are not
// merged in L2 (2000-byte bf16 rows: 3.5 TB/s streaming, 4.2 TB/s plain; 8000-byte
// rows: 5.4 against 5.0).  True when the rows of the tensor start and end on
// 64-byte boundaries.
template <typename T>
DEV bool rows_fill_lines(const Seg &s)
{
    return ((s.ptr | (uint64_t)(s.row_stride * Elem<T>::ESZ) | (uint64_t)((int64_t)s.n * Elem<T>::ESZ)) & 63u) == 0;
}

// Any strides; also the path of rows whose scale is outside the range of the
// fast exact division (plain IEEE divide, one element per lane and step).
template <typename T, int TEAM>
DEV void dequantize_gen(const Seg &s, const KParams &p, int row, int lane)
{
    if (row >= s.m) return;
    GLOBAL const uint8_t *in = as_global<const uint8_t>(p.packed + row_addr(s, p.slot_size, row));
    const DivCoef c = make_div(as_f(*(GLOBAL const u32 *)in));  // no zero guard (:239)
    const uint64_t base = s.ptr;
    const int64_t r0 = (int64_t)row * s.row_stride;
    if (c.fast) {
        for (int col = lane; col < s.n; col += TEAM) {
            const float f = __builtin_amdgcn_cvt_f32_fp8((int)in[4 + col], 0);
            Elem<T>::store(base, r0 + (int64_t)col * s.col_stride, div_fast_signed(f, c.r, c.r_lo));
        }
    } else {
#pragma nounroll
        for (int col = lane; col < s.n; col += TEAM) {
            const float f = __builtin_amdgcn_cvt_f32_fp8((int)in[4 + col], 0);
            Elem<T>::store(base, r0 + (int64_t)col * s.col_stride, f / c.s);
        }
    }
}

// Contiguous, 16-byte aligned rows.  Four vectors per lane and step; their loads
// are issued together without a branch (lanes past the end re-read the last
// vector and do not store).
template <typename T, int TEAM, bool NT>
DEV void dequantize_vec_nt(const Seg &s, const KParams &p, int row, int lane)
{
    if (row >= s.m) return;
    GLOBAL const u32 *in = as_global<const u32>(p.packed + row_addr(s, p.slot_size, row));
    const DivCoef c = make_div(as_f(in[0]));
    if (!c.fast) {  // same for all lanes of the team
        dequantize_gen<T, TEAM>(s, p, row, lane);
        return;
    }
    constexpr int EPV = Elem<T>::EPV;
    constexpr int DV = 8;  // loads in flight per lane (4: 1.3 % slower on 4096-column bf16 rows)
    const int nvec = s.n / EPV;
    GLOBAL u32x4_a2 *out = as_global<u32x4_a2>(s.ptr + (int64_t)row * s.row_stride * Elem<T>::ESZ);
    // the few columns after the last whole vector, one element per lane
    for (int col = nvec * EPV + lane; col < s.n; col += TEAM) {
        const float f = __builtin_amdgcn_cvt_f32_fp8((int)((GLOBAL const uint8_t *)in)[4 + col], 0);
        Elem<T>::store(s.ptr, (int64_t)row * s.row_stride + col, div_fast_signed(f, c.r, c.r_lo));
    }
    for (int base = 0; base < nvec; base += DV * TEAM) {
        u32x2 w[DV];
#pragma unroll
        for (int k = 0; k < DV; k++) {
            const int idx = min(base + k * TEAM + lane, nvec - 1);
            if constexpr (EPV == 4) {
                w[k].x = LOAD_STREAM(in + 1 + idx);
                w[k].y = 0;
            } else {
                w[k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)(in + 1 + 2 * idx));
            }
        }
#pragma unroll
        for (int k = 0; k < DV; k++) {
            const int idx = base + k * TEAM + lane;
            float o[EPV];
            float f[4];
            unpack_fp8x4(w[k].x, f);
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = div_fast_signed(f[e], c.r, c.r_lo);
            if constexpr (EPV == 8) {
                unpack_fp8x4(w[k].y, f);
#pragma unroll
                for (int e = 0; e < 4; e++) o[4 + e] = div_fast_signed(f[e], c.r, c.r_lo);
            }
            if (idx < nvec) {
                if (NT) STORE_STREAM(Elem<T>::pack(o), out + idx);
                else out[idx] = Elem<T>::pack(o);
            }
        }
    }
}

template <typename T, int TEAM>
DEV void dequantize_vec(const Seg &s, const KParams &p, int row, int lane)
{
    // same branch for the whole workgroup
    if (rows_fill_lines<T>(s)) dequantize_vec_nt<T, TEAM, true>(s, p, row, lane);
    else dequantize_vec_nt<T, TEAM, false>(s, p, row, lane);
}

// Rows of one column: one plain divide per row, four rows per lane.
template <typename T>
DEV void dequantize_col1(const Seg &s, const KParams &p, int row0, int tid)
{
    u32x2 w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int row = min(row0 + k * TFTQ_WG + tid, s.m - 1);
        w[k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)as_global<const u32>(p.packed + row_addr(s, p.slot_size, row)));
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int row = row0 + k * TFTQ_WG + tid;
        const float f = __builtin_amdgcn_cvt_f32_fp8((int)w[k].y, 0);
        if (row < s.m) Elem<T>::store(s.ptr, (int64_t)row * s.row_stride, f / as_f(w[k].x));  // no zero guard (:239)
    }
}

// K_VECS in dequantize: same shape as quantize_small, 8 vectors of codes and their
// rows' scales in flight per lane.
template <typename T, int LC, bool NT>
DEV void dequantize_small_c(const Seg &s, const KParams &p, int blk, int tid, const SmallShape &h)
{
    constexpr int EPV = Elem<T>::EPV;
    constexpr int C = 1 << LC, ROWS = 8 >> LC;
    const int nvec = s.n / EPV;
    const int row0 = blk * (h.teams * ROWS);
    const float inv = 1.0f / (float)s.slice_rows;

    u32x2 w[ROWS][C];
    float sc[ROWS];
    int row[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        row[r] = row0 + r * h.teams + h.t;
        GLOBAL const u32 *in =
            as_global<const u32>(p.packed + row_addr_fast(s, p.slot_size, min(row[r], s.m - 1), inv));
        sc[r] = as_f(in[0]);
#pragma unroll
        for (int k = 0; k < C; k++) {
            const int idx = min(k * h.team + h.l, nvec - 1);
            if constexpr (EPV == 4) {
                w[r][k].x = LOAD_STREAM(in + 1 + idx);
                w[r][k].y = 0;
            } else {
                w[r][k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)(in + 1 + 2 * idx));
            }
        }
    }
    bool all_fast = true;
#pragma unroll
    for (int r = 0; r < ROWS; r++) all_fast = all_fast && scale_is_fast(sc[r]);
    const bool fast = __builtin_amdgcn_ballot_w64(!all_fast) == 0;  // one code path per wavefront
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const DivCoef c = make_div(sc[r]);
        GLOBAL u32x4_a2 *out = as_global<u32x4_a2>(s.ptr + (int64_t)min(row[r], s.m - 1) * s.row_stride * Elem<T>::ESZ);
#pragma unroll
        for (int k = 0; k < C; k++) {
            float f[4], g[4], o[EPV];
            unpack_fp8x4(w[r][k].x, f);
            unpack_fp8x4(w[r][k].y, g);
            if (fast) {
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = div_fast_signed(f[e], c.r, c.r_lo);
                if constexpr (EPV == 8) {
#pragma unroll
                    for (int e = 0; e < 4; e++) o[4 + e] = div_fast_signed(g[e], c.r, c.r_lo);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = f[e] / sc[r];  // :250-252
                if constexpr (EPV == 8) {
#pragma unroll
                    for (int e = 0; e < 4; e++) o[4 + e] = g[e] / sc[r];
                }
            }
            const int vec = k * h.team + h.l;
            if (row[r] < s.m && vec < nvec) {
                if (NT) STORE_STREAM(Elem<T>::pack(o), out + vec);
                else out[vec] = Elem<T>::pack(o);
            }
        }
    }
}

template <typename T>
DEV void dequantize_small(const Seg &s, const KParams &p, int blk, int tid)
{
    const SmallShape h = small_shape(s.n / Elem<T>::EPV, tid);
    if (rows_fill_lines<T>(s)) {
        if (h.lc == 0) dequantize_small_c<T, 0, true>(s, p, blk, tid, h);
        else if (h.lc == 1) dequantize_small_c<T, 1, true>(s, p, blk, tid, h);
        else dequantize_small_c<T, 2, true>(s, p, blk, tid, h);
    } else {
        if (h.lc == 0) dequantize_small_c<T, 0, false>(s, p, blk, tid, h);
        else if (h.lc == 1) dequantize_small_c<T, 1, false>(s, p, blk, tid, h);
        else dequantize_small_c<T, 2, false>(s, p, blk, tid, h);
    }
}

template <typename T, bool INLINE>
__global__ __launch_bounds__(TFTQ_WG) void k_dequantize(const KParams p, const InlineTable inl)
{
    Seg s;
    int vb;
    if (!locate<INLINE, ST_D>(p, inl, s, vb)) return;
    const int blk = vb - s.wg_begin[ST_D];
    const int tid = threadIdx.x;
    switch (s.kind[ST_D]) {
    case K_VEC256: dequantize_vec<T, 256>(s, p, blk, tid); break;
    case K_VEC64:
        dequantize_vec<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_VEC32: dequantize_vec<T, 32>(s, p, blk * 8 + (tid >> 5), tid & 31); break;
    case K_VEC16: dequantize_vec<T, 16>(s, p, blk * 16 + (tid >> 4), tid & 15); break;
    case K_VEC8: dequantize_vec<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN64:
        dequantize_gen<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_GEN8: dequantize_gen<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN1: dequantize_gen<T, 1>(s, p, blk * 256 + tid, 0); break;
    case K_COL1:
        if (s.m > 0) dequantize_col1<T>(s, p, blk * 4 * TFTQ_WG, tid);
        break;
    case K_VECS: dequantize_small<T>(s, p, blk, tid); break;
    default: break;
    }
}

// ---------------------------------------------------------------------------
// reduce
// ---------------------------------------------------------------------------
// Loads dwords [d0, d0+4) of a row payload (ndw dwords long); dwords past the
// end read as 0 and are never touched in memory.  Codes past column n inside
// the last dword are cleared: the reference masks them (:420-424).
DEV u32x4 load_codes(GLOBAL const u32 *payload, int d0, int ndw, int n)
{
    u32x4 w = {0, 0, 0, 0};
    const int rem = ndw - d0;
    if (rem >= 4) {
        w = *(GLOBAL const u32x4_a4 *)(payload + d0);
    } else if (rem > 0) {
        w.x = payload[d0];
        if (rem > 1) w.y = payload[d0 + 1];
        if (rem > 2) w.z = payload[d0 + 2];
    }
    if (n & 3) {
        const int last = ndw - 1 - d0;
        const u32 mask = (1u << (8 * (n & 3))) - 1u;
        if (last == 0) w.x &= mask;
        if (last == 1) w.y &= mask;
        if (last == 2) w.z &= mask;
        if (last == 3) w.w &= mask;
    }
    return w;
}

DEV void store_codes(GLOBAL u32 *payload, int d0, int ndw, const u32x4 w)
{
    const int rem = ndw - d0;
    if (rem >= 4) {
        *(GLOBAL u32x4_a4 *)(payload + d0) = w;
    } else if (rem > 0) {
        payload[d0] = w.x;
        if (rem > 1) payload[d0 + 1] = w.y;
        if (rem > 2) payload[d0 + 2] = w.z;
    }
}

// acc[e] += code[e] / s for the 16 codes of w, s given as (r, r_lo)
DEV void accumulate16(float (&acc)[16], const u32x4 w, float r, float r_lo)
{
    const u32 ww[4] = {w.x, w.y, w.z, w.w};

#pragma unroll
    for (int t = 0; t < 4; t++) {
        float f[4];
        unpack_fp8x4(ww[t], f);
#pragma unroll
        for (int e = 0; e < 4; e++) acc[4 * t + e] = acc[4 * t + e] + div_fast(f[e], r, r_lo);
    }
}

// (acc * s2) / div, left to right (:364).  GDIV: div is not a power of two
// and needs a real divide; otherwise inv_div (1 for SUM) is an exact inverse
// and multiplying by it is the same correctly rounded result.
template <bool GDIV>
DEV float scale_div(float a, float s2, const KParams &p)
{
    const float y = a * s2;
    return GDIV ? y / p.div : y * p.inv_div;
}

template <bool GDIV>
DEV u32x4 requant16(const float (&a)[16], float s2, const KParams &p)
{
    float y[16];
#pragma unroll
    for (int e = 0; e < 16; e++) y[e] = scale_div<GDIV>(a[e], s2, p);
    u32x4 o;
    o.x = pack_fp8x4(y[0], y[1], y[2], y[3]);
    o.y = pack_fp8x4(y[4], y[5], y[6], y[7]);
    o.z = pack_fp8x4(y[8], y[9], y[10], y[11]);
    o.w = pack_fp8x4(y[12], y[13], y[14], y[15]);
    return o;
}

DEV GLOBAL const u32 *peer_row(const KParams &p, int k, int64_t off)
{
    int peer = p.rank + k;  // :407
    if (peer >= p.ws) peer -= p.ws;

    return as_global<const u32>(p.packed + (int64_t)peer * p.slot_size + off);
}

DEV float guarded_scale(GLOBAL const u32 *prow)
{
    const float sc = as_f(prow[0]);
    return sc == 0.0f ? 1.0f : sc;  // padding rows (:419)
}

// One column at a time with plain IEEE divides, two passes: the path of rows
// in which some peer's scale is outside the range of the fast exact division,
// and of rows too long for registers.  Small code, not tuned.
template <int TEAM, bool GDIV>
DEV void reduce_row_slow(const Seg &s, const KParams &p, int j, int lane, float *lds)
{
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    GLOBAL uint8_t *orow = as_global<uint8_t>(p.packed + (int64_t)p.rank * p.slot_size + off);
    float amax = 0.0f, s2 = 0.0f;
#pragma nounroll
    for (int pass = 0; pass < 2; pass++) {
#pragma nounroll
        for (int c = lane; c < s.n; c += TEAM) {
            float a = 0.0f;
#pragma nounroll
            for (int k = 0; k < p.ws; k++) {
                GLOBAL const u32 *prow = peer_row(p, k, off);
                const float sc = guarded_scale(prow);
                const int code = ((GLOBAL const uint8_t *)prow)[4 + c];
                a = a + __builtin_amdgcn_cvt_f32_fp8(code, 0) / sc;
            }
            if (pass == 0) {
                amax = fmaxf(amax, __builtin_fabsf(a));
            } else {
                const float y = scale_div<GDIV>(a, s2, p);
                orow[4 + c] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, 0.0f, 0, false) & 0xFF);
            }
        }
        if (pass == 0) {
            amax = team_max<TEAM>(amax, lds);
            s2 = calc_scale(amax / p.div);
        }
    }
    // the own slot's old scale is an input of every lane: write the new one last (:375)
    __threadfence_block();
    if (TEAM == 256) __syncthreads();
    if (lane == 0) *(GLOBAL u32 *)orow = as_u(s2);
}

// Rows longer than a 256-lane team can keep in registers (more than 16384
// columns): two passes over chunks of 1024 dwords, as the reference does for
// every row (:318-372), but with 16-byte loads, the fast exact division and the
// scales read once.  The second pass finds the peer rows in the caches.
template <bool GDIV>
DEV void reduce_row_long(const Seg &s, const KParams &p, int j, int tid, float *lds)
{
    const int ndw = (s.row_bytes >> 2) - 1;
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    const int wlane = tid & 63;
    const int ws = p.ws;  // <= 64 here
    const DivCoef c = make_div(guarded_scale(peer_row(p, min(wlane, ws - 1), off)));
    if (__builtin_amdgcn_ballot_w64(!c.fast) != 0) {  // same in the four wavefronts
        reduce_row_slow<256, GDIV>(s, p, j, tid, lds);
        return;
    }
    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
    const u32 tailmask = (s.n & 3) ? (1u << (8 * (s.n & 3))) - 1u : 0xFFFFFFFFu;
    float amax = 0.0f, s2 = 0.0f;
#pragma nounroll
    for (int pass = 0; pass < 2; pass++) {
#pragma nounroll
        for (int d = 0; d < ndw; d += 4 * TFTQ_WG) {
            const bool valid = d + 4 * tid < ndw;
            const int doff = min(d + 4 * tid, ndw - 4);  // the last vector ends with the row
            const u32 mask = doff == ndw - 4 ? tailmask : 0xFFFFFFFFu;
            float acc[16];
#pragma unroll
            for (int e = 0; e < 16; e++) acc[e] = 0.0f;
#pragma nounroll
            for (int k0 = 0; k0 < ws; k0 += 4) {
                u32x4 w[4];
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    w[b] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(peer_row(p, min(k0 + b, ws - 1), off) + 1 + doff));
                }
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    w[b].w &= mask;
                    if (k0 + b < ws) accumulate16(acc, w[b], bcast_lane(c.r, k0 + b), bcast_lane(c.r_lo, k0 + b));
                }
            }
            if (pass == 0) {
#pragma unroll
                for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[e]));
            } else {
                // the moved-back last vector overlaps its neighbour, which may sit in another
                // wavefront: nobody stores before everybody has read the own slot's chunk
                __syncthreads();
                if (valid) {
                    const u32x4 o = requant16<GDIV>(acc, s2, p);
                    if (doff >= d) {
                        *(GLOBAL u32x4_a4 *)(orow + 1 + doff) = o;
                    } else {
                        // The vector reaches back into the previous chunk, whose codes have
                        // already been replaced in the own slot: what was accumulated for
                        // those dwords is meaningless and they are final already.
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (doff + e >= d) orow[1 + doff + e] = o[e];
                    }
                }
            }
        }
        if (pass == 0) {
            amax = team_max<256>(amax, lds);  // every wavefront has read the old scales by now
            s2 = calc_scale(amax / p.div);
        }
    }
    if (tid == 0) orow[0] = as_u(s2);  // :375
}

// Register-resident row: the team holds all accumulators of the row, each peer
// row is read once.  UNITS = 16-byte vectors of codes per lane and peer.
template <int TEAM, int UNITS, bool GDIV>
DEV void reduce_row(const Seg &s, const KParams &p, int j, int lane, float *lds)
{
    constexpr int PB = 8 / UNITS;  // peers whose loads are in flight together
    if (j >= s.slice_rows) return;  // a team leaves whole: its lanes share the row
    const int ndw = (s.row_bytes >> 2) - 1;
    const int n = s.n;
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    const int wlane = threadIdx.x & 63;

    float acc[UNITS][16];
#pragma unroll
    for (int u = 0; u < UNITS; u++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[u][e] = 0.0f;

    for (int kc = 0; kc < p.ws; kc += 64) {
        const int kend = min(p.ws, kc + 64);
        // Wide teams: lane l of every wavefront fetches the scale of peer kc + l
        // first, then the codes of the first peers go in flight, and only then
        // are the scales turned into division coefficients.
        float my_scale = 1.0f;
        if (TEAM >= 64 && kc + wlane < p.ws) my_scale = guarded_scale(peer_row(p, kc + wlane, off));

        u32x4 w[PB][UNITS];
        float sraw[PB];
        auto load_batch = [&](int k0) {
#pragma unroll
            for (int b = 0; b < PB; b++) {
                if (k0 + b < kend) {
                    GLOBAL const u32 *prow = peer_row(p, k0 + b, off);
                    if (TEAM < 64) sraw[b] = guarded_scale(prow);
#pragma unroll
                    for (int u = 0; u < UNITS; u++)
                        w[b][u] = load_codes(prow + 1, (u * TEAM + lane) * 4, ndw, n);
                }
            }
        };
        load_batch(kc);

        float cr = 1.0f, cl = 0.0f;
        if (TEAM >= 64) {
            const DivCoef c = make_div(my_scale);
            cr = c.r;
            cl = c.r_lo;
            if (__builtin_amdgcn_ballot_w64(!c.fast) != 0) {  // some peer needs the plain divide
                reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);
                return;
            }
        }
        for (int k0 = kc; k0 < kend; k0 += PB) {
            if (k0 != kc) load_batch(k0);
            if (TEAM < 64) {
                bool fast = true;
#pragma unroll
                for (int b = 0; b < PB; b++)
                    if (k0 + b < kend) fast = fast && scale_is_fast(sraw[b]);
                if (!fast) {  // same decision in every lane of the team
                    reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);
                    return;
                }
            }
#pragma unroll
            for (int b = 0; b < PB; b++) {
                if (k0 + b < kend) {
                    float pr, pl;
                    if (TEAM >= 64) {
                        pr = bcast_lane(cr, k0 + b - kc);
                        pl = bcast_lane(cl, k0 + b - kc);
                    } else {
                        const DivCoef c = make_div(sraw[b]);
                        pr = c.r;
                        pl = c.r_lo;
                    }
#pragma unroll
                    for (int u = 0; u < UNITS; u++) accumulate16(acc[u], w[b][u], pr, pl);
                }
            }
        }
    }

    float amax = 0.0f;
#pragma unroll
    for (int u = 0; u < UNITS; u++)
#pragma unroll
        for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[u][e]));
    amax = team_max<TEAM>(amax, lds);
    const float s2 = calc_scale(amax / p.div);  // :340

    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
#pragma unroll
    for (int u = 0; u < UNITS; u++)
        store_codes(orow + 1, (u * TEAM + lane) * 4, ndw, requant16<GDIV>(acc[u], s2, p));
    // Every lane read the old scale of the own slot before team_max (wide
    // teams synchronise there; narrow teams are one wavefront in program order).
    if (lane == 0) orow[0] = as_u(s2);  // :375
}

// Several rows per team, software-pipelined: the codes of the next batch of
// peers (of this row or of the next row) are in flight while the current batch
// is accumulated, so a wavefront always has loads outstanding.  A batch is
// R_VPB 16-byte vectors per lane: R_VPB / UNITS peers of one row.  Loads carry
// no branch: a lane past the end of the row re-reads the row's last vector, a
// batch past the last peer re-reads the last peer, and both are ignored later.
// Needs ws <= min(TEAM, 64) (lane l of a team, or of each of its wavefronts,
// holds the scale of peer l) and rows of at least one 16-byte vector.  Teams
// smaller than a wavefront take one row each; a team whose row is past the end
// (`valid` false) works on the last row and stores nothing, so that the
// wavefront stays converged for the cross-lane operations.
constexpr int R_VPB = 4;

template <int TEAM, int UNITS, bool PIPE, bool GDIV>
DEV void reduce_rows(const Seg &s, const KParams &p, int j0, int nrows, int lane, float *lds, bool valid = true)
{
    constexpr int PB = R_VPB / UNITS >= 1 ? R_VPB / UNITS : 1;  // peers per batch
    if (TEAM >= 64 && nrows <= 0) return;
    const int ndw = (s.row_bytes >> 2) - 1;  // >= 4 here
    const int ws = p.ws;
    const int nb = (ws + PB - 1) / PB;  // batches per row
    const int total = nrows * nb;
    const int wlane = TEAM >= 64 ? (int)(threadIdx.x & 63u) : lane;
    const int speer = min(wlane, ws - 1);  // the peer whose scale this lane fetches

    // Vector u of this lane starts at dword doff[u].  The last vector of a row whose
    // length is not a multiple of 4 dwords is moved back so that it ends with the row:
    // it overlaps its neighbour, both lanes compute and store the same values.  Lanes
    // past the row's end re-read the last vector and do not store.
    int doff[UNITS];
    u32 padmask[UNITS];  // clears the bytes past column n in the row's last dword (:420-424)
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        doff[u] = min(4 * (u * TEAM + lane), ndw - 4);
        padmask[u] = (doff[u] == ndw - 4 && (s.n & 3)) ? (1u << (8 * (s.n & 3))) - 1u : 0xFFFFFFFFu;
    }

    struct Batch {
        u32x4 w[PB][UNITS];
        float scale;  // lane l: guarded scale of peer min(l, ws-1) of the batch's row
    };
    Batch A, B;

    int lrow = 0, lbatch = 0;  // next batch to load
    auto issue = [&](Batch &dst) {
        const int64_t off = s.slot_off + (int64_t)(j0 + lrow) * s.row_bytes;
        dst.scale = as_f(peer_row(p, speer, off)[0]);
#pragma unroll
        for (int b = 0; b < PB; b++) {
            GLOBAL const u32 *pv = peer_row(p, min(lbatch * PB + b, ws - 1), off) + 1;
#pragma unroll
            for (int u = 0; u < UNITS; u++)
                dst.w[b][u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + doff[u]));
        }
        if (++lbatch == nb) {
            lbatch = 0;
            ++lrow;
        }
    };

    float acc[UNITS][16];
#pragma unroll
    for (int u = 0; u < UNITS; u++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[u][e] = 0.0f;
    int crow = 0, cbatch = 0;  // batch being consumed
    float cr = 1.0f, cl = 0.0f;
    bool row_fast = true;

    auto consume = [&](const Batch &src) {
        if (cbatch == 0) {
            const float sc = src.scale == 0.0f ? 1.0f : src.scale;  // padding rows (:419)
            const DivCoef c = make_div(sc);
            cr = c.r;
            cl = c.r_lo;
            row_fast = __builtin_amdgcn_ballot_w64(!c.fast) == 0;  // same in all wavefronts of the team
        }
        if (row_fast) {
#pragma unroll
            for (int b = 0; b < PB; b++) {
                const int k = cbatch * PB + b;
                if (k < ws) {
                    const float pr = team_bcast<TEAM>(cr, k), pl = team_bcast<TEAM>(cl, k);
#pragma unroll
                    for (int u = 0; u < UNITS; u++) {
                        u32x4 w = src.w[b][u];
                        w.w &= padmask[u];  // here, not at the load: the load must stay in flight
                        accumulate16(acc[u], w, pr, pl);
                    }
                }
            }
        }
        if (++cbatch == nb) {
            const int j = j0 + crow;
            if (row_fast) {
                float amax = 0.0f;  // duplicates held by lanes past the row's end do not change it
#pragma unroll
                for (int u = 0; u < UNITS; u++)
#pragma unroll
                    for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[u][e]));
                amax = team_max<TEAM>(amax, lds);
                const float s2 = calc_scale(amax / p.div);  // :340
                const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
                GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
#pragma unroll
                for (int u = 0; u < UNITS; u++) {
                    const u32x4 o = requant16<GDIV>(acc[u], s2, p);
                    if (valid && 4 * (u * TEAM + lane) < ndw) *(GLOBAL u32x4_a4 *)(orow + 1 + doff[u]) = o;
                }
                if (valid && lane == 0) orow[0] = as_u(s2);  // :375; all lanes read the old scale before team_max
            } else if (valid) {
                reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);  // some peer needs the plain divide
            }
#pragma unroll
            for (int u = 0; u < UNITS; u++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[u][e] = 0.0f;
            cbatch = 0;
            ++crow;
        }
    };

    if (!PIPE) {  // long rows: one batch in flight keeps the register count down
        for (int i = 0; i < total; i++) {
            issue(A);
            consume(A);
        }
        return;
    }
    issue(A);
    int i = 0;
    for (; i + 2 < total; i += 2) {
        issue(B);
        consume(A);
        issue(A);
        consume(B);
    }
    if (i + 1 < total) {
        issue(B);
        consume(A);
        consume(B);
    } else {
        consume(A);
    }
}

// Rows of one column: 8 bytes per row and peer, one plain divide per peer
// (coefficients for the fast division would cost two), four rows per lane.
template <bool GDIV>
DEV void reduce_col1(const Seg &s, const KParams &p, int j0, int tid)
{
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    int64_t off[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        off[k] = s.slot_off + (int64_t)min(j0 + k * TFTQ_WG + tid, s.slice_rows - 1) * 8;
#pragma nounroll
    for (int kk = 0; kk < p.ws; kk++) {
        u32x2 w[4];
#pragma unroll
        for (int k = 0; k < 4; k++) w[k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)peer_row(p, kk, off[k]));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float sc = as_f(w[k].x);
            sc = sc == 0.0f ? 1.0f : sc;  // padding rows (:419)
            acc[k] = acc[k] + __builtin_amdgcn_cvt_f32_fp8((int)w[k].y, 0) / sc;
        }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        if (j0 + k * TFTQ_WG + tid < s.slice_rows) {
            const float s2 = calc_scale(__builtin_fabsf(acc[k]) / p.div);
            u32x2 o;
            o.x = as_u(s2);
            o.y = pack_fp8x4(scale_div<GDIV>(acc[k], s2, p), 0.0f, 0.0f, 0.0f) & 0xFFu;
            *(GLOBAL u32x2_a4 *)as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off[k]) = o;
        }
    }
}

template <bool INLINE, bool GDIV, bool WIDE>
__global__ __launch_bounds__(TFTQ_WG) void k_reduce(const KParams p, const InlineTable inl)
{
    __shared__ float lds[4];
    Seg s;
    int vb;
    if (!locate<INLINE, ST_R>(p, inl, s, vb)) return;
    const int blk = vb - s.wg_begin[ST_R];
    const int tid = threadIdx.x;
    const int ndw = (s.row_bytes >> 2) - 1;
    const int rpt = s.reduce_rows_per_team;
    switch (s.kind[ST_R]) {
    case K_GEN256: {
        const int j0 = blk * rpt;
        const int nrows = min(rpt, s.slice_rows - j0);
        if (WIDE && ndw > TFTQ_R_DWORDS && ndw <= TFTQ_R_DWORDS_WIDE && p.ws <= 64) {
            reduce_rows<256, 8, false, GDIV>(s, p, j0, nrows, tid, lds);
        } else if (ndw > TFTQ_R_DWORDS) {
            for (int r = 0; r < nrows; r++) {
                if (p.ws > 64) reduce_row_slow<256, GDIV>(s, p, j0 + r, tid, lds);
                else reduce_row_long<GDIV>(s, p, j0 + r, tid, lds);
            }
        } else if (p.ws > 64) {
            for (int r = 0; r < nrows; r++) {
                if (ndw <= 1024) reduce_row<256, 1, GDIV>(s, p, j0 + r, tid, lds);
                else reduce_row<256, 4, GDIV>(s, p, j0 + r, tid, lds);
            }
        } else if (ndw <= 1024) {
            reduce_rows<256, 1, true, GDIV>(s, p, j0, nrows, tid, lds);
        } else if (ndw <= 2048) {
            reduce_rows<256, 2, true, GDIV>(s, p, j0, nrows, tid, lds);
        } else {
            reduce_rows<256, 4, false, GDIV>(s, p, j0, nrows, tid, lds);
        }
        break;
    }
    case K_GEN64: {
        const int j0 = (blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6)) * rpt;
        const int nrows = min(rpt, s.slice_rows - j0);
        if (p.ws > 64) {
            for (int r = 0; r < nrows; r++) {
                if (ndw <= 256) reduce_row<64, 1, GDIV>(s, p, j0 + r, tid & 63, lds);
                else reduce_row<64, 2, GDIV>(s, p, j0 + r, tid & 63, lds);
            }
        } else if (ndw <= 256) {
            reduce_rows<64, 1, true, GDIV>(s, p, j0, nrows, tid & 63, lds);
        } else {
            reduce_rows<64, 2, true, GDIV>(s, p, j0, nrows, tid & 63, lds);
        }
        break;
    }
    case K_GEN32:
    case K_GEN16:
    case K_GEN8: {
        // one row per team of 32, 16 or 8 lanes
        auto small = [&](auto team_c) {
            constexpr int TEAM = decltype(team_c)::value;
            const int j = blk * (TFTQ_WG / TEAM) + tid / TEAM;
            if (p.ws <= TEAM) {
                reduce_rows<TEAM, 1, true, GDIV>(s, p, min(j, s.slice_rows - 1), 1, tid % TEAM, lds, j < s.slice_rows);
            } else {
                reduce_row<TEAM, 1, GDIV>(s, p, j, tid % TEAM, lds);
            }
        };
        if (s.kind[ST_R] == K_GEN32) small(std::integral_constant<int, 32>());
        else if (s.kind[ST_R] == K_GEN16) small(std::integral_constant<int, 16>());
        else small(std::integral_constant<int, 8>());
        break;
    }
    case K_GEN1:  // one lane per row: 1, 2 or 4 vectors of codes per peer
        if (ndw <= 4) reduce_row<1, 1, GDIV>(s, p, blk * 256 + tid, 0, lds);
        else if (ndw <= 8) reduce_row<1, 2, GDIV>(s, p, blk * 256 + tid, 0, lds);
        else reduce_row<1, 4, GDIV>(s, p, blk * 256 + tid, 0, lds);
        break;
    case K_COL1: reduce_col1<GDIV>(s, p, blk * 4 * TFTQ_WG, tid); break;
    default: break;
    }
}

// ---------------------------------------------------------------------------
// C ABI: launches
// ---------------------------------------------------------------------------
extern "C" int tftq_check_device(void)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    const char *a = prop.gcnArchName;
    return (a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0')
               ? 0
               : TFTQ_E_ARCH;
}

static void work_mapping(const tftq_plan *plan, int stage, KParams *kp)
{
    if (plan->nseg <= TFTQ_N_INLINE) {
        kp->dealt = plan->dealt[stage];
        kp->per_xcd = plan->dealt_per_xcd[stage];
        kp->map_shift = kp->chunk_shift = 0;
        kp->sorted_off = kp->map_off = 0;
    } else {
        kp->per_xcd = plan->index[stage].per_xcd;
        kp->map_shift = plan->index[stage].shift;
        kp->chunk_shift = plan->index[stage].chunk_shift;
        kp->sorted_off = plan->index[stage].sorted_off;
        kp->map_off = plan->index[stage].map_off;
    }
}

static int fill_params(const tftq_plan *plan, int stage, void *packed, int64_t packed_bytes,
                       KParams *kp, InlineTable *inl, bool *use_inline)
{
    if (!plan || !packed) return TFTQ_E_ARG;
    if (packed_bytes != plan->output_size) return TFTQ_E_SIZE;
    if (((uintptr_t)packed & 3) != 0) return TFTQ_E_ARG;
    *use_inline = plan->nseg <= TFTQ_N_INLINE;
    if (!*use_inline && !plan->device_table) return TFTQ_E_NOTABLE;
    kp->table = *use_inline ? nullptr : (const Seg *)plan->device_table;
    kp->packed = (uint8_t *)packed;
    kp->slot_size = plan->slot_size;
    kp->nseg = plan->nseg;
    kp->nwg = plan->nwg[stage];
    kp->ws = plan->ws;
    work_mapping(plan, stage, kp);
    kp->rank = 0;
    kp->div_mode = 0;
    kp->div = 1.0f;
    kp->inv_div = 1.0f;
    if (*use_inline)
        for (int i = 0; i < plan->nseg; i++) inl->s[i] = plan->segs[(size_t)i];
    return 0;
}

static inline unsigned grid_of(const KParams &kp)
{
    return (unsigned)(8 * kp.per_xcd);
}

template <typename T>
static int launch_q(const KParams &kp, const InlineTable &inl, bool use_inline, bool wide, hipStream_t st)
{
    const dim3 grid(grid_of(kp)), block(TFTQ_WG);
    if (wide) {
        if (use_inline) hipLaunchKernelGGL((k_quantize<T, true, true>), grid, block, 0, st, kp, inl);
        else hipLaunchKernelGGL((k_quantize<T, false, true>), grid, block, 0, st, kp, inl);
    } else {
        if (use_inline) hipLaunchKernelGGL((k_quantize<T, true, false>), grid, block, 0, st, kp, inl);
        else hipLaunchKernelGGL((k_quantize<T, false, false>), grid, block, 0, st, kp, inl);
    }
    return (int)hipGetLastError();
}

template <typename T>
static int launch_d(const KParams &kp, const InlineTable &inl, bool use_inline, hipStream_t st)
{
    if (use_inline)
        hipLaunchKernelGGL((k_dequantize<T, true>), dim3(grid_of(kp)), dim3(TFTQ_WG), 0, st, kp, inl);
    else
        hipLaunchKernelGGL((k_dequantize<T, false>), dim3(grid_of(kp)), dim3(TFTQ_WG), 0, st, kp, inl);
    return (int)hipGetLastError();
}

extern "C" int tftq_quantize(const tftq_plan *plan, void *packed, int64_t packed_bytes, void *stream)
{
    KParams kp;
    InlineTable inl = {};
    bool use_inline;
    int rc = fill_params(plan, ST_Q, packed, packed_bytes, &kp, &inl, &use_inline);
    if (rc) return rc;
    for (int i = 0; i < plan->nseg; i++)
        if (plan->segs[(size_t)i].ptr == 0 && plan->segs[(size_t)i].m > 0 && plan->segs[(size_t)i].n > 0)
            return TFTQ_E_ARG;
    if (kp.nwg == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    switch (plan->dtype) {
    case TFTQ_F32: return launch_q<float>(kp, inl, use_inline, plan->wide[ST_Q], st);
    case TFTQ_F16: return launch_q<f16_tag>(kp, inl, use_inline, plan->wide[ST_Q], st);
    case TFTQ_BF16: return launch_q<bf16_tag>(kp, inl, use_inline, plan->wide[ST_Q], st);
    default: return TFTQ_E_DTYPE;
    }
}

extern "C" int tftq_dequantize(const tftq_plan *plan, const void *packed, int64_t packed_bytes,
                               void *stream)
{
    KParams kp;
    InlineTable inl = {};
    bool use_inline;
    int rc = fill_params(plan, ST_D, (void *)packed, packed_bytes, &kp, &inl, &use_inline);
    if (rc) return rc;
    for (int i = 0; i < plan->nseg; i++)
        if (plan->segs[(size_t)i].ptr == 0 && plan->segs[(size_t)i].m > 0 && plan->segs[(size_t)i].n > 0)
            return TFTQ_E_ARG;
    if (kp.nwg == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    switch (plan->dtype) {
    case TFTQ_F32: return launch_d<float>(kp, inl, use_inline, st);
    case TFTQ_F16: return launch_d<f16_tag>(kp, inl, use_inline, st);
    case TFTQ_BF16: return launch_d<bf16_tag>(kp, inl, use_inline, st);
    default: return TFTQ_E_DTYPE;
    }
}

extern "C" int tftq_reduce(const tftq_plan *plan, void *packed, int64_t packed_bytes, int rank,
                           int is_avg, void *stream)
{
    KParams kp;
    InlineTable inl = {};
    bool use_inline;
    int rc = fill_params(plan, ST_R, packed, packed_bytes, &kp, &inl, &use_inline);
    if (rc) return rc;
    if (rank < 0 || rank >= plan->ws) return TFTQ_E_ARG;
    kp.rank = rank;
    if (is_avg) {
        const int ws = plan->ws;
        kp.div = (float)ws;
        if ((ws & (ws - 1)) == 0) {
            kp.div_mode = 1;
            kp.inv_div = 1.0f / (float)ws;
        } else {
            kp.div_mode = 2;
        }
    }
    if (kp.nwg == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(grid_of(kp)), block(TFTQ_WG);
    const bool gdiv = kp.div_mode == 2;
#define TFTQ_LAUNCH_R(I, G, W) hipLaunchKernelGGL((k_reduce<I, G, W>), grid, block, 0, st, kp, inl)
    if (plan->wide[ST_R]) {
        if (gdiv) { if (use_inline) TFTQ_LAUNCH_R(true, true, true); else TFTQ_LAUNCH_R(false, true, true); }
        else { if (use_inline) TFTQ_LAUNCH_R(true, false, true); else TFTQ_LAUNCH_R(false, false, true); }
    } else {
        if (gdiv) { if (use_inline) TFTQ_LAUNCH_R(true, true, false); else TFTQ_LAUNCH_R(false, true, false); }
        else { if (use_inline) TFTQ_LAUNCH_R(true, false, false); else TFTQ_LAUNCH_R(false, false, false); }
    }
#undef TFTQ_LAUNCH_R
    return (int)hipGetLastError();
}
