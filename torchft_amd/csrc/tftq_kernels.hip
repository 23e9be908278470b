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

#include "../../include/tftq.h"
#include "tftq_internal.h"

typedef uint32_t u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x2 u32x2_a4 __attribute__((aligned(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct bf16_tag {};
struct f16_tag {};

#define DEV __device__ __forceinline__
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
    if (TEAM >= 64) {
        v = fmaxf(v, dpp_mov<0x140>(v));  // row_mirror: all 16 lanes of a row agree
        const float a = bcast_lane(v, 0), b = bcast_lane(v, 16);
        const float c = bcast_lane(v, 32), d = bcast_lane(v, 48);
        v = fmaxf(fmaxf(a, b), fmaxf(c, d));
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
// Consecutive workgroup ids are dealt round-robin to the 8 XCDs.  Give XCD x
// the x-th contiguous eighth of the work instead.  The grid is launched with
// 8 * ceil(nwg / 8) workgroups; ids that map past nwg return -1.
DEV int virtual_block(int nwg)
{
    const int per_xcd = (nwg + 7) >> 3;
    const int vb = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    return vb < nwg ? vb : -1;
}

template <bool INLINE, int STAGE>
DEV Seg find_seg(const KParams &p, const InlineTable &inl, int vb)
{
    if (INLINE) {
        int i = p.nseg - 1;
        while (i > 0 && inl.s[i].wg_begin[STAGE] > vb) --i;
        return inl.s[i];
    } else {
        // last segment with wg_begin <= vb
        int lo = 0, hi = p.nseg - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (p.table[mid].wg_begin[STAGE] <= vb) lo = mid; else hi = mid - 1;
        }
        return p.table[lo];
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
        *(GLOBAL u32x2_a4 *)(payload + 2 * idx) = o;
    }
}

// Contiguous, 16-byte aligned rows of at most TEAM * QV vectors.
template <typename T, int TEAM>
DEV void quantize_vec(const Seg &s, const KParams &p, int row, int lane, float *lds)
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
    GLOBAL const u32x4 *in = as_global<const u32x4>(s.ptr + (int64_t)row * s.row_stride * Elem<T>::ESZ);
    u32x4 v[QV];
#pragma unroll
    for (int k = 0; k < QV; k++) {
        const int idx = k * TEAM + lane;
        const u32x4 z = {0, 0, 0, 0};
        v[k] = idx < nvec ? __builtin_nontemporal_load(in + idx) : z;
    }
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < QV; k++) amax = fmaxf(amax, vec_absmax<T>(v[k]));
    amax = team_max<TEAM>(amax, lds);
    const float sc = calc_scale(amax);
    if (lane == 0) out[0] = as_u(sc);
#pragma unroll
    for (int k = 0; k < QV; k++) {
        const int idx = k * TEAM + lane;
        if (idx < nvec) vec_quant_store<T>(v[k], sc, out + 1, idx);
    }
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

template <typename T, bool INLINE>
__global__ __launch_bounds__(TFTQ_WG) void k_quantize(const KParams p, const InlineTable inl)
{
    __shared__ float lds[4];
    const int vb = virtual_block(p.nwg);
    if (vb < 0) return;
    const Seg s = find_seg<INLINE, ST_Q>(p, inl, vb);
    const int blk = vb - s.wg_begin[ST_Q];
    const int tid = threadIdx.x;
    switch (s.kind[ST_Q]) {
    case K_VEC256: quantize_vec<T, 256>(s, p, blk, tid, lds); break;
    case K_VEC64:
        quantize_vec<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63, lds);
        break;
    case K_VEC8: quantize_vec<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7, lds); break;
    case K_GEN64:
        quantize_gen<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_GEN8: quantize_gen<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN1: quantize_gen<T, 1>(s, p, blk * 256 + tid, 0); break;
    default: break;
    }
}

// ---------------------------------------------------------------------------
// dequantize
// ---------------------------------------------------------------------------
template <typename T>
DEV u32x4 dequant_vec_unit(GLOBAL const u32 *payload, int idx, float r, float r_lo)
{
    constexpr int EPV = Elem<T>::EPV;
    float o[EPV];
    if constexpr (EPV == 4) {
        float f[4];
        unpack_fp8x4(payload[idx], f);
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = div_fast_signed(f[e], r, r_lo);
    } else {
        const u32x2 w = *(GLOBAL const u32x2_a4 *)(payload + 2 * idx);
        float f[4], g[4];
        unpack_fp8x4(w.x, f);
        unpack_fp8x4(w.y, g);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            o[e] = div_fast_signed(f[e], r, r_lo);
            o[4 + e] = div_fast_signed(g[e], r, r_lo);
        }
    }
    return Elem<T>::pack(o);
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

template <typename T, int TEAM>
DEV void dequantize_vec(const Seg &s, const KParams &p, int row, int lane)
{
    if (row >= s.m) return;
    GLOBAL const u32 *in = as_global<const u32>(p.packed + row_addr(s, p.slot_size, row));
    const DivCoef c = make_div(as_f(in[0]));
    if (!c.fast) {  // same for all lanes of the team
        dequantize_gen<T, TEAM>(s, p, row, lane);
        return;
    }
    const int nvec = s.n / Elem<T>::EPV;
    GLOBAL u32x4 *out = as_global<u32x4>(s.ptr + (int64_t)row * s.row_stride * Elem<T>::ESZ);
#pragma unroll 4
    for (int idx = lane; idx < nvec; idx += TEAM)
        out[idx] = dequant_vec_unit<T>(in + 1, idx, c.r, c.r_lo);
}

template <typename T, bool INLINE>
__global__ __launch_bounds__(TFTQ_WG) void k_dequantize(const KParams p, const InlineTable inl)
{
    const int vb = virtual_block(p.nwg);
    if (vb < 0) return;
    const Seg s = find_seg<INLINE, ST_D>(p, inl, vb);
    const int blk = vb - s.wg_begin[ST_D];
    const int tid = threadIdx.x;
    switch (s.kind[ST_D]) {
    case K_VEC256: dequantize_vec<T, 256>(s, p, blk, tid); break;
    case K_VEC64:
        dequantize_vec<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_VEC8: dequantize_vec<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN64:
        dequantize_gen<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_GEN8: dequantize_gen<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN1: dequantize_gen<T, 1>(s, p, blk * 256 + tid, 0); break;
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

    // can every peer's scale take the fast exact division?
    bool all_fast = true;
    if (TEAM >= 64) {
        for (int k = wlane; k < p.ws; k += 64)
            all_fast = all_fast && scale_is_fast(guarded_scale(peer_row(p, k, off)));
        all_fast = __builtin_amdgcn_ballot_w64(!all_fast) == 0;
    } else {
        for (int k = 0; k < p.ws; k++)
            all_fast = all_fast && scale_is_fast(guarded_scale(peer_row(p, k, off)));
    }
    if (!all_fast) {
        reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);
        return;
    }

    float acc[UNITS][16];
#pragma unroll
    for (int u = 0; u < UNITS; u++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[u][e] = 0.0f;

    for (int kc = 0; kc < p.ws; kc += 64) {
        // wide teams: lane l of every wavefront prepares peer kc + l
        float cr = 1.0f, cl = 0.0f;
        if (TEAM >= 64 && kc + wlane < p.ws) {
            const DivCoef c = make_div(guarded_scale(peer_row(p, kc + wlane, off)));
            cr = c.r;
            cl = c.r_lo;
        }
        const int kend = min(p.ws, kc + 64);
        for (int k0 = kc; k0 < kend; k0 += PB) {
            u32x4 w[PB][UNITS];
            float sraw[PB];
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

template <bool INLINE, bool GDIV>
__global__ __launch_bounds__(TFTQ_WG) void k_reduce(const KParams p, const InlineTable inl)
{
    __shared__ float lds[4];
    const int vb = virtual_block(p.nwg);
    if (vb < 0) return;
    const Seg s = find_seg<INLINE, ST_R>(p, inl, vb);
    const int blk = vb - s.wg_begin[ST_R];
    const int tid = threadIdx.x;
    const int ndw = (s.row_bytes >> 2) - 1;
    switch (s.kind[ST_R]) {
    case K_GEN256:
        if (ndw <= 1024) reduce_row<256, 1, GDIV>(s, p, blk, tid, lds);
        else if (ndw <= 4096) reduce_row<256, 4, GDIV>(s, p, blk, tid, lds);
        else reduce_row_slow<256, GDIV>(s, p, blk, tid, lds);
        break;
    case K_GEN64:
        reduce_row<64, 1, GDIV>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63, lds);
        break;
    case K_GEN8: reduce_row<8, 1, GDIV>(s, p, blk * 32 + (tid >> 3), tid & 7, lds); break;
    case K_GEN1: reduce_row<1, 1, GDIV>(s, p, blk * 256 + tid, 0, lds); break;
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
    kp->rank = 0;
    kp->div_mode = 0;
    kp->div = 1.0f;
    kp->inv_div = 1.0f;
    if (*use_inline)
        for (int i = 0; i < plan->nseg; i++) inl->s[i] = plan->segs[(size_t)i];
    return 0;
}

static inline unsigned grid_of(int nwg) { return (unsigned)(((nwg + 7) / 8) * 8); }

template <typename T>
static int launch_q(const KParams &kp, const InlineTable &inl, bool use_inline, hipStream_t st)
{
    if (use_inline)
        hipLaunchKernelGGL((k_quantize<T, true>), dim3(grid_of(kp.nwg)), dim3(TFTQ_WG), 0, st, kp, inl);
    else
        hipLaunchKernelGGL((k_quantize<T, false>), dim3(grid_of(kp.nwg)), dim3(TFTQ_WG), 0, st, kp, inl);
    return (int)hipGetLastError();
}

template <typename T>
static int launch_d(const KParams &kp, const InlineTable &inl, bool use_inline, hipStream_t st)
{
    if (use_inline)
        hipLaunchKernelGGL((k_dequantize<T, true>), dim3(grid_of(kp.nwg)), dim3(TFTQ_WG), 0, st, kp, inl);
    else
        hipLaunchKernelGGL((k_dequantize<T, false>), dim3(grid_of(kp.nwg)), dim3(TFTQ_WG), 0, st, kp, inl);
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
    case TFTQ_F32: return launch_q<float>(kp, inl, use_inline, st);
    case TFTQ_F16: return launch_q<f16_tag>(kp, inl, use_inline, st);
    case TFTQ_BF16: return launch_q<bf16_tag>(kp, inl, use_inline, st);
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
    const dim3 grid(grid_of(kp.nwg)), block(TFTQ_WG);
    if (kp.div_mode == 2) {
        if (use_inline) hipLaunchKernelGGL((k_reduce<true, true>), grid, block, 0, st, kp, inl);
        else hipLaunchKernelGGL((k_reduce<false, true>), grid, block, 0, st, kp, inl);
    } else {
        if (use_inline) hipLaunchKernelGGL((k_reduce<true, false>), grid, block, 0, st, kp, inl);
        else hipLaunchKernelGGL((k_reduce<false, false>), grid, block, 0, st, kp, inl);
    }
    return (int)hipGetLastError();
}
