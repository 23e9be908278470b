// Device helpers and launch plumbing shared by the three kernel files
// (tftq_quantize.hip, tftq_reduce.hip, tftq_dequantize.hip): HIP kernels for
// gfx950 (MI355X) and the compute entry points of the C ABI.
//
// Three kernels, one launch per stage:
//   k_quantize<T>    fused_quantize_into_fp8   (torchft/quantization.py:53-162)
//   k_reduce         fused_reduce_fp8          (:261-428)
//   k_dequantize<T>  fused_dequantize_from_fp8 (:165-258)
//
// Design (none of it follows the reference's launch shape):
//   * a row is owned by a "team" of 1 to 256 lanes chosen from the row length
//     (so that a lane has about 8 loads of 16 bytes in flight; lanes of very
//     short rows work on several rows); the team loads the row once, keeps it in
//     registers, reduces |x| with DPP inside the wavefront (LDS across the four
//     wavefronts of a 256-lane team) and converts from registers with the
//     packed fp8 converts of gfx950.  Every stage reads HBM once.
//   * all tensors of a call are covered by one launch: a workgroup finds its
//     tensor in a table of 64-byte descriptors (in the kernel arguments for
//     short lists) and branches on the team size stored there.
//   * workgroup ids are remapped so that each of the 8 XCDs works on
//     contiguous pieces of every tensor (neighbouring packed rows share cache
//     lines), in reduce the tensors with the heaviest workgroups first.
//   * division by a row scale is exact IEEE division, computed as
//     fma(f, r, f * r_lo) with r = RN(1/s) and r_lo = RN(fma(-s, r, 1) / s).
//     For the 253 finite e4m3 values f and every binary32 s with exponent in
//     [-64, 64] this equals RN(f / s) bit for bit (checked exhaustively by
//     tests/test_exact_division.py); other scales take the plain divide.
//
// Build flags that matter: -ffp-contract=off (the arithmetic contract is
// separate IEEE multiply / divide / add), packed fp32 ops disabled.

#pragma once

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
typedef u32 u32_a2 __attribute__((aligned(2)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
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
    } else if constexpr (TEAM == 1) {
        return v;
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
    if (TEAM >= 2) v = fmaxf(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
    if (TEAM >= 4) v = fmaxf(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
    if (TEAM >= 8) v = fmaxf(v, dpp_mov<0x141>(v));  // row_half_mirror
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

// r_lo = RN(e / s) with e = fma(-s, r, 1), without a second divide: one Newton step on
// e * r gives the correctly rounded quotient for every scale in the fast range
// (tests/exact_division.c compares the two for all 2^23 mantissas); outside that range
// the coefficients are not used.
DEV DivCoef make_div(float s)
{
    DivCoef c;
    c.s = s;
    c.r = 1.0f / s;
    const float e = __builtin_fmaf(-s, c.r, 1.0f);
    const float lo = e * c.r;
    c.r_lo = __builtin_fmaf(__builtin_fmaf(-s, lo, e), c.r, lo);
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
    DEV static float rounded(float v) { return v; }  // v as a stored element reads back
    // elements idx and idx + 1 with one access (streaming: neighbouring lanes take neighbouring
    // pairs, so a wavefront covers whole lines)
    DEV static void load2(uint64_t base, int64_t idx, float &a, float &b)
    {
        const u32x2 w = LOAD_STREAM((GLOBAL const u32x2_a4 *)(as_global<const float>(base) + idx));
        a = as_f(w.x);
        b = as_f(w.y);
    }
    DEV static void store2(uint64_t base, int64_t idx, float a, float b)
    {
        const u32x2 w = {as_u(a), as_u(b)};
        STORE_STREAM(w, (GLOBAL u32x2_a4 *)(as_global<float>(base) + idx));
    }
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
    DEV static float rounded(float v) { return as_f(pack2(v, 0.0f) << 16); }
    DEV static void load2(uint64_t base, int64_t idx, float &a, float &b)
    {
        const u32 w = LOAD_STREAM((GLOBAL const u32_a2 *)(as_global<const uint16_t>(base) + idx));
        a = as_f(w << 16);
        b = as_f(w & 0xFFFF0000u);
    }
    DEV static void store2(uint64_t base, int64_t idx, float a, float b)
    {
        STORE_STREAM(pack2(a, b), (GLOBAL u32_a2 *)(as_global<uint16_t>(base) + idx));
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
    DEV static float rounded(float v) { return (float)(_Float16)opaque(v); }
    DEV static void load2(uint64_t base, int64_t idx, float &a, float &b)
    {
        unpack2(LOAD_STREAM((GLOBAL const u32_a2 *)(as_global<const uint16_t>(base) + idx)), a, b);
    }
    DEV static void store2(uint64_t base, int64_t idx, float a, float b)
    {
        STORE_STREAM(pack2(a, b), (GLOBAL u32_a2 *)(as_global<uint16_t>(base) + idx));
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
    int i = (int)(blockIdx.x >> 3);
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
        int natural = p.natural;
        asm volatile("" : "+s"(cum_end_), "+s"(base_), "+s"(seg_), "+s"(natural) : "s"(p.packed), "s"(p.slot_size), "s"(p.ws), "s"(p.rank));
        if (natural) i = (int)blockIdx.x;  // all eight rows of the table describe the whole work
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
        asm volatile("" ::"s"(p.table), "s"(p.ptrs), "s"(p.map_off), "s"(p.sorted_off), "s"(p.map_shift), "s"(p.chunk_shift),
                     "s"(p.nwg), "s"(p.pieces), "s"(p.packed), "s"(p.slot_size), "s"(p.ws), "s"(p.rank));
        // chunks of 2^chunk_shift consecutive workgroups go to the XCDs in turn
        const int cs = p.chunk_shift;
        vb = ((((i >> cs) << 3) + x) << cs) + (i & ((1 << cs) - 1));
        if (vb >= p.nwg) return false;
        if (STAGE == ST_R && p.pieces) {  // this wavefront's quarter of the workgroup (tftq_reduce_pieces)
            vb = 4 * vb + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
            if (vb >= p.pieces) return false;
        }
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
        // the table holds no addresses: the tensor's comes from the call's pointer array
        uint64_t tptr = 0;
        if (STAGE != ST_R) tptr = *(const CONSTANT uint64_t *)((uint64_t)p.ptrs + (uint64_t)sg * 8u);
        __builtin_memcpy(&s, v, sizeof(Seg));
        s.ptr = tptr;
        return true;
    }
}

DEV int64_t row_addr(const Seg &s, int64_t slot_size, int row)
{
    const int slot = row / s.slice_rows;
    const int j = row - slot * s.slice_rows;
    return (int64_t)slot * slot_size + s.slot_off + (int64_t)j * s.row_bytes;
}

// Short contiguous rows of whole 16-byte vectors (K_VECS; the shape is
// tftq_small_shape): 1 to 32 lanes per row, and every lane works on several rows
// so that it has 8 loads in flight.  Row slot r of team t is row
// row0 + r * teams + t: for a given r the teams of a wavefront read
// consecutive rows, i.e. consecutive memory.
struct SmallShape {
    int lt, c, team, teams, t, l;
};
DEV SmallShape small_shape(int nvec, int tid, int stage)
{
    SmallShape h;
    tftq_small_shape(nvec, &h.lt, &h.c, stage);
    h.team = 1 << h.lt;
    h.teams = TFTQ_WG >> h.lt;
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

// ---------------------------------------------------------------------------
// packed rows through LDS
// ---------------------------------------------------------------------------
// Staging of a workgroup's packed rows in LDS.  The rows that one workgroup quantizes are
// neighbours in the packed buffer, so together they are one span of bytes; packed rows
// start anywhere (4 + n bytes each), which makes direct stores cover parts of 128-byte
// lines with every instruction.  The workgroup instead assembles the span in LDS, at the
// offset that the span has inside its first 128-byte line, and then copies it out with
// streaming 16-byte stores whose wavefronts each cover eight whole lines; only the first
// and the last 16 bytes of the span can be partial and go out as halfwords.
#define LDS_AS __attribute__((address_space(3)))

DEV void copy_out_span(const uint8_t *stage, uint8_t *g0, int len, int tid)
{
    const int mis = (int)((uintptr_t)g0 & 127u);
    GLOBAL uint8_t *line0 = as_global<uint8_t>(g0 - mis);  // stage[x] belongs at line0[x]
    const int end = mis + len;
    const int nchunks = (end + 15) >> 4;
#pragma nounroll
    for (int c = tid; c < nchunks; c += TFTQ_WG) {
        const int lo = 16 * c;
        const u32x4 v = *(const LDS_AS u32x4 *)(const LDS_AS uint8_t *)(stage + lo);
        if (lo >= mis && lo + 16 <= end) {
            STORE_STREAM(v, (GLOBAL u32x4 *)(line0 + lo));
        } else {  // the span's first or last 16 bytes: halfwords (a span starts and ends at even bytes)
            const u32 w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int d = 0; d < 8; d++)
                if (lo + 2 * d >= mis && lo + 2 * d < end)
                    *(GLOBAL uint16_t *)(line0 + lo + 2 * d) = (uint16_t)(w[d >> 1] >> (16 * (d & 1)));
        }
    }
}

// ---------------------------------------------------------------------------
// host side: kernel parameters of a launch
// ---------------------------------------------------------------------------
static inline void work_mapping(const tftq_plan *plan, int stage, KParams *kp)
{
    if (plan->nseg <= TFTQ_N_INLINE) {
        kp->dealt = plan->dealt[stage];
        kp->per_xcd = plan->dealt_per_xcd[stage];
        kp->natural = plan->natural[stage] ? 1 : 0;
        kp->pieces = 0;
        kp->map_shift = kp->chunk_shift = 0;
        kp->sorted_off = kp->map_off = 0;
    } else {
        kp->per_xcd = plan->index[stage].per_xcd;
        kp->natural = 0;
        kp->pieces = plan->index[stage].pieces;
        kp->map_shift = plan->index[stage].shift;
        kp->chunk_shift = plan->index[stage].chunk_shift;
        kp->sorted_off = plan->index[stage].sorted_off;
        kp->map_off = plan->index[stage].map_off;
    }
}

// Makes `device` current for the lifetime of the object and restores the caller's device
// afterwards; device < 0 leaves the current device alone.
struct DeviceScope {
    int prev = -1;
    bool switched = false;
    hipError_t err = hipSuccess;
    explicit DeviceScope(int device)
    {
        if (device < 0) return;
        err = hipGetDevice(&prev);
        if (err == hipSuccess && prev != device) {
            err = hipSetDevice(device);
            switched = err == hipSuccess;
        }
    }
    ~DeviceScope()
    {
        if (switched) (void)hipSetDevice(prev);
    }
    DeviceScope(const DeviceScope &) = delete;
    DeviceScope &operator=(const DeviceScope &) = delete;
};

// Copies `bytes` bytes (a multiple of 8) from host memory to 8-byte aligned device memory
// with small kernels on `st` that carry the data in their arguments: the source is read
// before the function returns, nothing is allocated or synchronised, and a stream capture
// records the data itself.  Defined in tftq_runtime.hip.
__attribute__((visibility("hidden"))) int tftq_put_bytes(void *dst_device, const void *src_host, size_t bytes,
                                                         hipStream_t st);

// Looks up, for the current device, the address of the fixed array that tftq_reduce_static
// keeps its table in.  Defined in tftq_reduce.hip.
__attribute__((visibility("hidden"))) int tftq_static_table_setup(void);

// One kernel launch with the launch's own error (not whatever an earlier call left behind).
template <typename K>
static inline int launch_kernel(K kernel, unsigned grid, unsigned lds_bytes, hipStream_t st, const KParams &kp,
                                const InlineTable &inl)
{
    void *args[2] = {(void *)&kp, (void *)&inl};
    return (int)hipLaunchKernel((const void *)kernel, dim3(grid), dim3(TFTQ_WG), args, lds_bytes, st);
}

// Kernel parameters of one call.  tensors: host array of the tensors' device addresses (null
// in reduce); table / pointers: the caller's device buffers of a long list.  For a long list
// with `tensors` the addresses are written to `pointers` on `st` first.
static inline int fill_params(const tftq_plan *plan, int stage, const void *const *tensors, const void *table,
                              void *pointers, void *packed, int64_t packed_bytes, hipStream_t st, KParams *kp,
                              InlineTable *inl, bool *use_inline)
{
    if (!plan) return TFTQ_E_ARG;
    if (packed_bytes != plan->output_size) return TFTQ_E_SIZE;
    // a list of empty tensors has an empty packed buffer, whose address may be null
    if (!packed && plan->output_size != 0) return TFTQ_E_ARG;
    if (((uintptr_t)packed & 3) != 0) return TFTQ_E_ARG;
    *use_inline = plan->nseg <= TFTQ_N_INLINE;
    const bool needs_tensors = stage != ST_R && plan->nwg[stage] > 0;
    if (*use_inline) {
        if (needs_tensors && !tensors) return TFTQ_E_ARG;
        for (int i = 0; i < plan->nseg; i++) {
            inl->s[i] = plan->segs[(size_t)i];
            if (stage != ST_R) {
                inl->s[i].ptr = (uint64_t)(uintptr_t)(tensors ? tensors[i] : nullptr);
                if (inl->s[i].ptr == 0 && inl->s[i].m > 0 && inl->s[i].n > 0) return TFTQ_E_ARG;
            }
        }
    } else if (plan->nwg[stage] > 0) {
        if (!table || ((uintptr_t)table & 255) != 0) return TFTQ_E_NOTABLE;
        if (needs_tensors) {
            if (!pointers || ((uintptr_t)pointers & 7) != 0) return TFTQ_E_NOTABLE;
            if (tensors) {
                for (int i = 0; i < plan->nseg; i++)
                    if (!tensors[i] && plan->segs[(size_t)i].m > 0 && plan->segs[(size_t)i].n > 0) return TFTQ_E_ARG;
                const int rc = tftq_put_bytes(pointers, tensors, (size_t)plan->nseg * 8, st);
                if (rc) return rc;
            }
        }
    }
    kp->table = *use_inline ? nullptr : (const Seg *)table;
    kp->ptrs = (*use_inline || stage == ST_R) ? nullptr : (const uint64_t *)pointers;
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
    kp->post_scale = 1.0f;
    return 0;
}

static inline unsigned grid_of(const KParams &kp)
{
    return (unsigned)(8 * kp.per_xcd);
}
