// k_quantize and tftq_quantize: fused_quantize_into_fp8 on gfx950.
//
// Follows torchft/quantization.py:53-162 (kernel) and :531-588 (launcher); design notes in tftq_device.h.

#include "tftq_device.h"

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

// the 4 (fp32) or 8 (16-bit) codes of one input vector: one or two dwords
template <typename T>
DEV u32x2 vec_codes(const u32x4 v, float s)
{
    float f[Elem<T>::EPV];
    Elem<T>::unpack(v, f);
    u32x2 o = {0u, 0u};
    o.x = pack_fp8x4(f[0] * s, f[1] * s, f[2] * s, f[3] * s);
    if constexpr (Elem<T>::EPV == 8) o.y = pack_fp8x4(f[4] * s, f[5] * s, f[6] * s, f[7] * s);
    return o;
}

template <typename T>
DEV void vec_quant_store(const u32x4 v, float s, GLOBAL u32 *payload, int idx)
{
    const u32x2 o = vec_codes<T>(v, s);
    if constexpr (Elem<T>::EPV == 4) {
        payload[idx] = o.x;
    } else {
        *(GLOBAL u32x2_a4 *)(payload + 2 * idx) = o;  // plain store: rows start 4 bytes off a line, L2 merges
    }
}

// Lanes past the last vector of a row re-read its last vector, moved down to a 16-byte
// boundary when the row starts off one (the row has at least two vectors, so the bytes
// are still the row's): whole wavefronts of such lanes then cost one aligned access, while
// 64 copies of a vector at an odd 2-byte offset are served lane by lane (10001-column
// bf16 rows, five vectors per lane needed and eight loaded: 153.8 us against 117.1 us for 10000).
DEV int dup_vec_offset(GLOBAL const u32x4_a2 *in, int nvec)
{
    return (nvec - 1) * 16 - (int)((uintptr_t)in & 15u);
}
DEV GLOBAL const u32x4_a2 *vec_or_dup(GLOBAL const u32x4_a2 *in, int idx, int nvec, int dup)
{
    return (GLOBAL const u32x4_a2 *)((GLOBAL const uint8_t *)in + (idx < nvec ? idx * 16 : dup));
}

constexpr int Q_STAGE_BYTES = 16640;  // 8 rows of 2052 bytes (2048 16-bit columns) + 127 bytes of offset, rounded up (see copy_out_span)
// the wide kernel, whose three workgroups per CU leave each 53 KB of LDS: one row of 32768 16-bit columns
constexpr int Q_STAGE_BYTES_WIDE = 32912;

// Contiguous, 16-byte aligned rows of at most TEAM * KMAX vectors.  The KMAX
// loads of a lane are issued back to back without a branch in between: lanes
// past the end of the row re-read its last vector (a duplicate cannot change
// the maximum) and simply do not store.
// STAGED: the row is a real one and its packed image goes to LDS at srow (see copy_out_span).
template <typename T, int TEAM, int KMAX, bool STAGED = false>
DEV void quantize_vec_k(const Seg &s, const KParams &p, int row, int lane, float *lds, LDS_AS u32 *srow = nullptr)
{
    GLOBAL u32 *out = nullptr;
    if (!STAGED) {
        const bool active = row < s.slice_rows * p.ws;
        out = as_global<u32>(p.packed + (active ? row_addr(s, p.slot_size, row) : 0));
        if (active && row >= s.m) {
            // padding row: the reference leaves it zero (:93-95 on a zero-filled buffer)
            for (int d = lane; d < (s.row_bytes >> 2); d += TEAM) out[d] = 0;
        }
        if (!active || row >= s.m) return;  // a team leaves whole: its lanes share the row
    }

    constexpr int EPV = Elem<T>::EPV;
    const int nvec = s.n / EPV;
    const int tail = s.n - nvec * EPV;  // elements after the last whole vector (rare)
    const int64_t r0 = (int64_t)row * s.row_stride;
    GLOBAL const u32x4_a2 *in = as_global<const u32x4_a2>(s.ptr + r0 * Elem<T>::ESZ);
    const int dup = dup_vec_offset(in, nvec);
    u32x4 v[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; k++) v[k] = LOAD_STREAM(vec_or_dup(in, k * TEAM + lane, nvec, dup));
    // the few elements after the last whole vector: lane e of the team takes element e (the
    // lanes behind them re-read the last one), and later stores its code
    float te = 0.0f;
    if (tail) te = Elem<T>::load(s.ptr, r0 + nvec * EPV + min(lane, tail - 1));
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < KMAX; k++) amax = fmaxf(amax, vec_absmax<T>(v[k]));
    if (tail) amax = fmaxf(amax, __builtin_fabsf(te));
    amax = team_max<TEAM>(amax, lds);
    const float sc = calc_scale(amax);
    if (lane == 0) {
        if (STAGED) srow[0] = as_u(sc);
        else out[0] = as_u(sc);
    }
    // The elements are unpacked again from the raw vectors: keeping the floats of the
    // maximum search alive until here would double the registers of 16-bit inputs.
#pragma unroll
    for (int k = 0; k < KMAX; k++) asm volatile("" : "+v"(v[k].x), "+v"(v[k].y), "+v"(v[k].z), "+v"(v[k].w));
#pragma unroll
    for (int k = 0; k < KMAX; k++) {
        const int idx = k * TEAM + lane;
        if (idx < nvec) {
            if (STAGED) {
                const u32x2 o = vec_codes<T>(v[k], sc);
                if constexpr (EPV == 4) {
                    srow[1 + idx] = o.x;
                } else {
                    srow[1 + 2 * idx] = o.x;
                    srow[2 + 2 * idx] = o.y;
                }
            } else {
                vec_quant_store<T>(v[k], sc, out + 1, idx);
            }
        }
    }
    // tail codes and the zero pad bytes behind them, one byte per lane (a team has at least 8 lanes)
    if (tail && lane < s.row_bytes - 4 - nvec * EPV) {
        const u32 b = lane < tail ? pack_fp8x4(te * sc, 0.0f, 0.0f, 0.0f) & 0xFFu : 0u;
        const int at = 4 + nvec * EPV + lane;
        if (STAGED) ((LDS_AS uint8_t *)srow)[at] = (uint8_t)b;
        else ((GLOBAL uint8_t *)out)[at] = (uint8_t)b;
    }
}

// Rows of more than 4096 vectors (64 KB; wide kernel only): the first 16
// vectors of a lane stay in registers, up to 15 more are parked in LDS, where
// every lane reads back only what it wrote itself, so rows of up to 7936
// vectors (124 KB) are still read from memory once.  The parked vectors travel
// in three groups of five; the loads of the next group are issued before the
// current one is parked.  What a longer row has beyond 7936 vectors is read
// twice, once for the maximum and once to be quantized.
template <typename T>
DEV void quantize_vec_lds(const Seg &s, const KParams &p, int row, int tid, float *lds, u32x4 *park)
{
    constexpr int KR = 2 * QV, G = TFTQ_Q_PARK_GROUP, NG = TFTQ_Q_PARKED / G;
    static_assert(NG * G == TFTQ_Q_PARKED, "groups of five");
    const bool active = row < s.slice_rows * p.ws;
    GLOBAL u32 *out = as_global<u32>(p.packed + (active ? row_addr(s, p.slot_size, row) : 0));
    if (active && row >= s.m) {
        for (int d = tid; d < (s.row_bytes >> 2); d += TFTQ_WG) out[d] = 0;  // padding row
    }
    if (!active || row >= s.m) return;  // the whole workgroup leaves

    constexpr int EPV = Elem<T>::EPV;
    const int nvec = s.n / EPV;
    const int tail = s.n - nvec * EPV;
    const int64_t r0 = (int64_t)row * s.row_stride;
    GLOBAL const u32x4_a2 *in = as_global<const u32x4_a2>(s.ptr + r0 * Elem<T>::ESZ);
    const int dup = dup_vec_offset(in, nvec);
    u32x4 v[KR], w[2][G];
#pragma unroll
    for (int k = 0; k < KR; k++) v[k] = LOAD_STREAM(vec_or_dup(in, k * TFTQ_WG + tid, nvec, dup));
#pragma unroll
    for (int k = 0; k < G; k++) w[0][k] = LOAD_STREAM(vec_or_dup(in, (KR + k) * TFTQ_WG + tid, nvec, dup));
    float te = 0.0f;  // lane e takes element e behind the last whole vector (see quantize_vec_k)
    if (tail) te = Elem<T>::load(s.ptr, r0 + nvec * EPV + min(tid, tail - 1));
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < KR; k++) amax = fmaxf(amax, vec_absmax<T>(v[k]));
    // the groups this row needs (the launch has LDS for the longest row of the list)
    const int ng = tftq_q_park_groups(nvec);
#pragma unroll
    for (int g = 0; g < NG; g++) {
        if (g < ng) {  // same for the whole workgroup
            if (g + 1 < NG && g + 1 < ng) {
#pragma unroll
                for (int k = 0; k < G; k++)
                    w[(g + 1) & 1][k] = LOAD_STREAM(vec_or_dup(in, (KR + (g + 1) * G + k) * TFTQ_WG + tid, nvec, dup));
            }
#pragma unroll
            for (int k = 0; k < G; k++) {
                amax = fmaxf(amax, vec_absmax<T>(w[g & 1][k]));
                park[(g * G + k) * TFTQ_WG + tid] = w[g & 1][k];
            }
        }
    }
    if (tail) amax = fmaxf(amax, __builtin_fabsf(te));
#pragma nounroll
    for (int base = TFTQ_Q_VECS_LDS; base < nvec; base += 4 * TFTQ_WG) {  // first pass over the rest
        u32x4 x[4];
#pragma unroll
        for (int k = 0; k < 4; k++) x[k] = in[min(base + k * TFTQ_WG + tid, nvec - 1)];
#pragma unroll
        for (int k = 0; k < 4; k++) amax = fmaxf(amax, vec_absmax<T>(x[k]));
    }
    amax = team_max<256>(amax, lds);
    const float sc = calc_scale(amax);
    if (tid == 0) out[0] = as_u(sc);
#pragma unroll
    for (int k = 0; k < KR; k++) asm volatile("" : "+v"(v[k].x), "+v"(v[k].y), "+v"(v[k].z), "+v"(v[k].w));
#pragma unroll
    for (int k = 0; k < KR; k++) {
        const int idx = k * TFTQ_WG + tid;
        if (idx < nvec) vec_quant_store<T>(v[k], sc, out + 1, idx);
    }
#pragma unroll
    for (int k = 0; k < TFTQ_Q_PARKED; k++) {
        const int idx = (KR + k) * TFTQ_WG + tid;
        if (idx < nvec) vec_quant_store<T>(park[k * TFTQ_WG + tid], sc, out + 1, idx);
    }
#pragma nounroll
    for (int base = TFTQ_Q_VECS_LDS; base < nvec; base += 4 * TFTQ_WG) {  // second pass over the rest
        u32x4 x[4];
#pragma unroll
        for (int k = 0; k < 4; k++) x[k] = LOAD_STREAM(in + min(base + k * TFTQ_WG + tid, nvec - 1));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int idx = base + k * TFTQ_WG + tid;
            if (idx < nvec) vec_quant_store<T>(x[k], sc, out + 1, idx);
        }
    }
    if (tail && tid < s.row_bytes - 4 - nvec * EPV) {  // tail codes and the zero pad bytes behind them
        const u32 b = tid < tail ? pack_fp8x4(te * sc, 0.0f, 0.0f, 0.0f) & 0xFFu : 0u;
        ((GLOBAL uint8_t *)out)[4 + nvec * EPV + tid] = (uint8_t)b;
    }
}

template <typename T, int TEAM, bool WIDE>
DEV void quantize_vec(const Seg &s, const KParams &p, int row, int lane, float *lds, u32x4 *park)
{
    // same branch for the whole workgroup
    const int nvec = s.n / Elem<T>::EPV;
    if (nvec <= (QV / 2) * TEAM) quantize_vec_k<T, TEAM, QV / 2>(s, p, row, lane, lds);
    else if (TEAM < 256 || nvec <= TFTQ_Q_VECS) quantize_vec_k<T, TEAM, QV>(s, p, row, lane, lds);
    else if (WIDE && nvec <= TFTQ_Q_VECS_WIDE) quantize_vec_k<T, TEAM, 2 * QV>(s, p, row, lane, lds);
    else if (WIDE) quantize_vec_lds<T>(s, p, row, lane, lds, park);
    // else: the planner launches the wide kernel, with its LDS, for plans that have such rows
}

// The TFTQ_WG / TEAM rows of workgroup blk.  When they are all real rows of one slot (all
// but the workgroups at the end of a slot or of the tensor) and fit the staging buffer,
// their packed rows are assembled in LDS and written as one span; otherwise row by row.
template <typename T, int TEAM, bool WIDE>
DEV void quantize_vec_rows(const Seg &s, const KParams &p, int blk, int tid, float *lds, u32x4 *park, uint8_t *stage)
{
    constexpr int R = TFTQ_WG / TEAM;
    const int r0 = blk * R;
    const int team = TEAM == 64 ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid / TEAM;
    const int lane = tid & (TEAM - 1);
    {
        constexpr int KMAX = WIDE && TEAM == 256 ? 2 * QV : QV;  // vectors per lane that the kernel keeps in registers
        constexpr int STAGE_BYTES = WIDE ? Q_STAGE_BYTES_WIDE : Q_STAGE_BYTES;
        const int nvec = s.n / Elem<T>::EPV;
        const int last = r0 + R - 1;
        if (last < s.m && nvec <= KMAX * TEAM) {
            const int slot = r0 / s.slice_rows;
            const int j = r0 - slot * s.slice_rows;
            uint8_t *g0 = p.packed + (int64_t)slot * p.slot_size + s.slot_off + (int64_t)j * s.row_bytes;
            const int mis = (int)((uintptr_t)g0 & 127u);
            const int len = R * s.row_bytes;
            if (j + R <= s.slice_rows && mis + len <= STAGE_BYTES) {  // same for the whole workgroup
                LDS_AS u32 *srow = (LDS_AS u32 *)(LDS_AS uint8_t *)(stage + mis + team * s.row_bytes);
                if (nvec <= (QV / 2) * TEAM) quantize_vec_k<T, TEAM, QV / 2, true>(s, p, r0 + team, lane, lds, srow);
                else if (KMAX == QV || nvec <= QV * TEAM) quantize_vec_k<T, TEAM, QV, true>(s, p, r0 + team, lane, lds, srow);
                else quantize_vec_k<T, TEAM, KMAX, true>(s, p, r0 + team, lane, lds, srow);
                __syncthreads();
                copy_out_span(stage, g0, len, tid);
                return;
            }
        }
    }
    quantize_vec<T, TEAM, WIDE && TEAM == 256>(s, p, r0 + team, lane, lds, park);
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
// [scale, code] of one row
DEV u32x2 quantize_one(float x)
{
    // maximum with 0 as for longer rows: a NaN element is ignored (:131-143)
    const float sc = calc_scale(fmaxf(0.0f, __builtin_fabsf(x)));
    u32x2 o;
    o.x = as_u(sc);
    o.y = pack_fp8x4(x * sc, 0.0f, 0.0f, 0.0f) & 0xFFu;
    return o;
}

// Any element stride: four rows per lane, interleaved so that every 8-byte
// [scale, code] store of a wavefront is contiguous.
template <typename T>
DEV void quantize_col1_strided(const Seg &s, const KParams &p, int row0, int tid)
{
    const int m_pad = s.slice_rows * p.ws;
    const float inv = 1.0f / (float)s.slice_rows;
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
            if (row < s.m) o = quantize_one(x[k]);
            *(GLOBAL u32x2_a4 *)as_global<u32>(p.packed + row_addr_fast(s, p.slot_size, row, inv)) = o;
        }
    }
}

// Contiguous elements: a lane takes TFTQ_COL1_PAIRS_Q pairs of neighbouring rows, so that it
// reads two elements with one load (a wavefront reads 256 or 512 contiguous
// bytes per load even for 2-byte elements) and writes their two packed rows
// with one 16-byte streaming store (a wavefront writes 1 KB of whole lines).
// A pair that straddles the end of a slot or of the tensor is stored row by row.
template <typename T>
DEV void quantize_col1(const Seg &s, const KParams &p, int row0, int tid)
{
    if (s.row_stride != 1) {  // same for the whole workgroup
#pragma nounroll
        for (int r = 0; r < 2 * TFTQ_COL1_PAIRS_Q * TFTQ_WG && row0 + r < s.slice_rows * p.ws; r += 4 * TFTQ_WG)
            quantize_col1_strided<T>(s, p, row0 + r, tid);
        return;
    }
    const int m_pad = s.slice_rows * p.ws;
    const float inv = 1.0f / (float)s.slice_rows;
    float x[TFTQ_COL1_PAIRS_Q][2];
#pragma unroll
    for (int k = 0; k < TFTQ_COL1_PAIRS_Q; k++) {
        const int row = row0 + 2 * (k * TFTQ_WG + tid);
        x[k][0] = x[k][1] = 0.0f;
        if (row + 1 < s.m) Elem<T>::load2(s.ptr, row, x[k][0], x[k][1]);
        else if (row < s.m) x[k][0] = Elem<T>::load(s.ptr, row);
    }
#pragma unroll
    for (int k = 0; k < TFTQ_COL1_PAIRS_Q; k++) {
        const int row = row0 + 2 * (k * TFTQ_WG + tid);
        if (row >= m_pad) continue;
        u32x2 a = {0u, 0u}, b = {0u, 0u};  // padding rows stay zero
        if (row < s.m) a = quantize_one(x[k][0]);
        if (row + 1 < s.m) b = quantize_one(x[k][1]);
        int slot = (int)((float)row * inv);  // off by at most one
        int j = row - slot * s.slice_rows;
        if (j < 0) { --slot; j += s.slice_rows; }
        if (j >= s.slice_rows) { ++slot; j -= s.slice_rows; }
        GLOBAL u32 *dst = as_global<u32>(p.packed + (int64_t)slot * p.slot_size + s.slot_off + (int64_t)j * 8);
        if (j + 1 < s.slice_rows) {  // the next row follows in the same slot (and row + 1 < m_pad)
            const u32x4 o = {a.x, a.y, b.x, b.y};
            STORE_STREAM(o, (GLOBAL u32x4_a4 *)dst);
        } else {
            *(GLOBAL u32x2_a4 *)dst = a;
            if (row + 1 < m_pad)
                *(GLOBAL u32x2_a4 *)as_global<u32>(p.packed + row_addr_fast(s, p.slot_size, row + 1, inv)) = b;
        }
    }
}

// Short contiguous rows of 1 to 32 16-byte vectors (K_VECS, shape in tftq_device.h).  A row
// whose length is not a whole number of vectors has its last vector moved back so that it
// ends with the row: it overlaps its neighbour, whose elements count twice for the maximum
// (no matter) and whose codes are written twice with the same values.
// First column of vector idx of a row of n columns.
template <typename T>
DEV int small_vec_col(int idx, int n)
{
    return min(idx * Elem<T>::EPV, n - Elem<T>::EPV);
}

DEV void put8(LDS_AS uint8_t *q, u32 v) { *q = (uint8_t)v; }
DEV void put8(GLOBAL uint8_t *q, u32 v) { *q = (uint8_t)v; }
DEV void put32(LDS_AS uint8_t *q, u32 v) { *(LDS_AS u32 *)q = v; }
DEV void put32(GLOBAL uint8_t *q, u32 v) { *(GLOBAL u32 *)q = v; }
DEV void put64(LDS_AS uint8_t *q, u32x2 v) { *(LDS_AS u32x2_a4 *)q = v; }
DEV void put64(GLOBAL uint8_t *q, u32x2 v) { *(GLOBAL u32x2_a4 *)q = v; }

// The codes o of vector idx (of nv) into the packed row at `row` (LDS or global memory); the
// lane of the last vector also clears the pad bytes behind the row's last code.
// TAIL false: rows of whole vectors, which have neither a moved vector nor pad bytes.
template <typename T, bool TAIL, typename P>
DEV void put_small_codes(P row, int idx, int nv, int n, int row_bytes, const u32x2 o)
{
    constexpr int EPV = Elem<T>::EPV;
    if constexpr (!TAIL) {
        if constexpr (EPV == 4) put32(row + 4 + idx * EPV, o.x);
        else put64(row + 4 + idx * EPV, o);
        return;
    }
    const int col = small_vec_col<T>(idx, n);
    if ((col & 3) == 0) {
        if constexpr (EPV == 4) put32(row + 4 + col, o.x);
        else put64(row + 4 + col, o);
    } else {  // the moved last vector of a row that is not a whole number of dwords
#pragma unroll
        for (int e = 0; e < EPV; e++) put8(row + 4 + col + e, (e < 4 ? o.x : o.y) >> (8 * (e & 3)));
    }
    if (idx == nv - 1)
        for (int b = 4 + n; b < row_bytes; b++) put8(row + b, 0u);
}

// Scale of the row whose vectors a lane holds in v (maximum over the lanes of its team).
template <typename T, int C>
DEV float small_row_scale(const u32x4 (&v)[C], const SmallShape &h)
{
    float a = 0.0f;
#pragma unroll
    for (int k = 0; k < C; k++) {
        a = fmaxf(a, vec_absmax<T>(v[k]));
    }
    if (h.lt >= 1) a = fmaxf(a, dpp_mov<0xB1>(a));   // quad_perm [1,0,3,2]
    if (h.lt >= 2) a = fmaxf(a, dpp_mov<0x4E>(a));   // quad_perm [2,3,0,1]
    if (h.lt >= 3) a = fmaxf(a, dpp_mov<0x141>(a));  // row_half_mirror
    if (h.lt >= 4) a = fmaxf(a, dpp_mov<0x140>(a));  // row_mirror: all 16 lanes of a row agree
    if (h.lt >= 5) {  // same for the whole workgroup
        const float lo = fmaxf(bcast_lane(a, 0), bcast_lane(a, 16)), hi = fmaxf(bcast_lane(a, 32), bcast_lane(a, 48));
        a = (threadIdx.x & 32) ? hi : lo;
    }
    return calc_scale(a);
}

// Rows RBEG * teams .. REND * teams - 1 of the workgroup's rows (those up to `last`)
// through the LDS stage: g0 is the address of the workgroup's first packed row.
template <typename T, int C, bool TAIL, int RBEG, int REND>
DEV void quantize_small_span(const Seg &s, const SmallShape &h, const u32x4 (&v)[8 / C][C], int row0, int last,
                             uint8_t *g0, uint8_t *stage, int tid)
{
    const int nvec = tftq_small_nvec(s.n, Elem<T>::ESZ);
    const int first = row0 + RBEG * h.teams;
    if (first > last) return;  // same for the whole workgroup
    uint8_t *gp = g0 + (int64_t)(RBEG * h.teams) * s.row_bytes;
    const int mis = (int)((uintptr_t)gp & 127u);
    const int len = (min(last, row0 + REND * h.teams - 1) - first + 1) * s.row_bytes;
#pragma unroll
    for (int r = RBEG; r < REND; r++) {
        const int row = row0 + r * h.teams + h.t;
        const float sc = small_row_scale<T, C>(v[r], h);
        if (row > last) continue;
        LDS_AS uint8_t *srow = (LDS_AS uint8_t *)(stage + mis + ((r - RBEG) * h.teams + h.t) * s.row_bytes);
        if (row >= s.m) {  // padding row: zero (:93-95 on a zero-filled buffer)
            for (int d = h.l; d < (s.row_bytes >> 2); d += h.team) ((LDS_AS u32 *)srow)[d] = 0;
            continue;
        }
        if (h.l == 0) *(LDS_AS u32 *)srow = as_u(sc);
#pragma unroll
        for (int k = 0; k < C; k++) {
            const int idx = k * h.team + h.l;
            if (idx >= nvec) continue;
            const u32x4 x = v[r][k];
            put_small_codes<T, TAIL>(srow, idx, nvec, s.n, s.row_bytes, vec_codes<T>(x, sc));
        }
    }
    __syncthreads();
    copy_out_span(stage, gp, len, tid);
}

// The rows of a workgroup are neighbours; when they lie in one slot their packed rows are
// one span of bytes, which goes through LDS (copy_out_span) in two halves (rows of 8 to 64
// 16-bit columns make up to 24 KB per workgroup, more than the stage holds).
template <typename T, int C, bool TAIL>
DEV void quantize_small_c(const Seg &s, const KParams &p, int blk, int tid, const SmallShape &h, uint8_t *stage)
{
    constexpr int ROWS = 8 / C;  // C vectors per lane and row, ROWS rows per lane: 8 or 4
    const int nvec = tftq_small_nvec(s.n, Elem<T>::ESZ);
    const int nrows = h.teams * ROWS;
    const int row0 = blk * nrows;
    const int m_pad = s.slice_rows * p.ws;
    const float inv = 1.0f / (float)s.slice_rows;

    u32x4 v[ROWS][C];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int row = row0 + r * h.teams + h.t;
        const int64_t e0 = (int64_t)min(row, s.m - 1) * s.row_stride;  // s.m >= 1: there are rows
        // a lane past the row's last vector re-reads that one: a duplicate cannot change the maximum
        if constexpr (TAIL) {
#pragma unroll
            for (int k = 0; k < C; k++) {
                const int col = small_vec_col<T>(min(k * h.team + h.l, nvec - 1), s.n);
                v[r][k] = LOAD_STREAM(as_global<const u32x4_a2>(s.ptr + (e0 + col) * Elem<T>::ESZ));
            }
        } else {
            GLOBAL const u32x4_a2 *in = as_global<const u32x4_a2>(s.ptr + e0 * Elem<T>::ESZ);
#pragma unroll
            for (int k = 0; k < C; k++) v[r][k] = LOAD_STREAM(in + min(k * h.team + h.l, nvec - 1));
        }
    }
    {
        // the workgroup's rows that exist, row0 .. last, and the slot of the first one
        const int last = min(row0 + nrows, m_pad) - 1;
        int slot0 = (int)((float)row0 * inv);
        int j0 = row0 - slot0 * s.slice_rows;
        if (j0 < 0) { --slot0; j0 += s.slice_rows; }
        if (j0 >= s.slice_rows) { ++slot0; j0 -= s.slice_rows; }
        if (j0 + (last - row0) < s.slice_rows) {  // one slot: one span.  Same for the whole workgroup
            // the marker keeps the compiler from moving what this path and the one below have in
            // common, the scales of all rows, in front of the branch (20 more registers)
            asm volatile("; rows through the stage");
            uint8_t *g0 = p.packed + (int64_t)slot0 * p.slot_size + s.slot_off + (int64_t)j0 * s.row_bytes;
            quantize_small_span<T, C, TAIL, 0, ROWS / 2>(s, h, v, row0, last, g0, stage, tid);
            __syncthreads();  // the first half has been copied out of the stage
            quantize_small_span<T, C, TAIL, ROWS / 2, ROWS>(s, h, v, row0, last, g0, stage, tid);
            return;
        }
    }
    asm volatile("; rows straight from the registers");
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int row = row0 + r * h.teams + h.t;
        const float sc = small_row_scale<T, C>(v[r], h);
        if (row >= m_pad) continue;
        GLOBAL uint8_t *out = as_global<uint8_t>(p.packed + row_addr_fast(s, p.slot_size, row, inv));
        if (row >= s.m) {
            // padding row: the reference leaves it zero (:93-95 on a zero-filled buffer)
            for (int d = h.l; d < (s.row_bytes >> 2); d += h.team) ((GLOBAL u32 *)out)[d] = 0;
            continue;
        }
        if (h.l == 0) *(GLOBAL u32 *)out = as_u(sc);
#pragma unroll
        for (int k = 0; k < C; k++) {
            const int idx = k * h.team + h.l;
            if (idx >= nvec) continue;
            const u32x4 x = v[r][k];
            put_small_codes<T, TAIL>(out, idx, nvec, s.n, s.row_bytes, vec_codes<T>(x, sc));
        }
    }
}

template <typename T>
DEV void quantize_small(const Seg &s, const KParams &p, int blk, int tid, uint8_t *stage)
{
    const SmallShape h = small_shape(tftq_small_nvec(s.n, Elem<T>::ESZ), tid, ST_Q);
    // one or two vectors per lane (tftq_small_shape); same branch for the whole workgroup
    if (s.n % Elem<T>::EPV) {
        if (h.c == 1) quantize_small_c<T, 1, true>(s, p, blk, tid, h, stage);
        else quantize_small_c<T, 2, true>(s, p, blk, tid, h, stage);
    } else if (h.c == 1) quantize_small_c<T, 1, false>(s, p, blk, tid, h, stage);
    else quantize_small_c<T, 2, false>(s, p, blk, tid, h, stage);
}

template <typename T, bool INLINE, bool WIDE>
// The wide variant is held to 128 registers (four waves per SIMD instead of three at the 153 to
// 166 it would take): lists that mix rows of more than 32 KB with shorter ones run whole in
// it, and the shorter rows gain 10 % (a Llama-3-70B layer bucket: 464 -> 420 us).
__global__ __launch_bounds__(TFTQ_WG, WIDE ? 4 : 1) void k_quantize(const KParams p, const InlineTable inl)
{
    __shared__ float lds[4];
    __shared__ __align__(16) uint8_t stage_regular[WIDE ? 16 : Q_STAGE_BYTES];  // see copy_out_span
    // Dynamic LDS of the wide kernel: Q_STAGE_BYTES_WIDE as its stage, or the 40 or 60 KB that the
    // longest row of the plan parks there (which limits a CU to three or two workgroups); a
    // workgroup uses it for one or the other.
    extern __shared__ u32x4 park[];
    uint8_t *stage = WIDE ? (uint8_t *)park : stage_regular;
    Seg s;
    int vb;
    if (!locate<INLINE, ST_Q>(p, inl, s, vb)) return;
    const int blk = vb - s.wg_begin[ST_Q];
    const int tid = threadIdx.x;
    switch (s.kind[ST_Q]) {
    case K_VEC256: quantize_vec_rows<T, 256, WIDE>(s, p, blk, tid, lds, park, stage); break;
    case K_VEC64: quantize_vec_rows<T, 64, WIDE>(s, p, blk, tid, lds, park, stage); break;
    case K_VEC32: quantize_vec_rows<T, 32, WIDE>(s, p, blk, tid, lds, park, stage); break;
    case K_VEC16: quantize_vec_rows<T, 16, WIDE>(s, p, blk, tid, lds, park, stage); break;
    case K_VEC8: quantize_vec_rows<T, 8, WIDE>(s, p, blk, tid, lds, park, stage); break;
    case K_GEN64:
        quantize_gen<T, 64>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_GEN8: quantize_gen<T, 8>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN1: quantize_gen<T, 1>(s, p, blk * 256 + tid, 0); break;
    case K_COL1: quantize_col1<T>(s, p, blk * tftq_col1_rows_per_wg(ST_Q), tid); break;
    case K_VECS: quantize_small<T>(s, p, blk, tid, stage); break;
    default: break;
    }
}

template <typename T>
static int launch_q(const KParams &kp, const InlineTable &inl, bool use_inline, bool wide, int parked,
                    hipStream_t st)
{
    const unsigned grid = grid_of(kp);
    if (wide) {
        // the parking area also serves as the stage
        const unsigned lds = std::max((unsigned)parked * TFTQ_Q_PARK_GROUP * TFTQ_WG * 16u, (unsigned)Q_STAGE_BYTES_WIDE);
        if (use_inline) return launch_kernel(k_quantize<T, true, true>, grid, lds, st, kp, inl);
        return launch_kernel(k_quantize<T, false, true>, grid, lds, st, kp, inl);
    }
    if (use_inline) return launch_kernel(k_quantize<T, true, false>, grid, 0, st, kp, inl);
    return launch_kernel(k_quantize<T, false, false>, grid, 0, st, kp, inl);
}

extern "C" int tftq_quantize(const tftq_plan *plan, const void *const *tensors, const void *table,
                             void *pointers, void *packed, int64_t packed_bytes, int device, void *stream)
{
    KParams kp;
    InlineTable inl = {};
    bool use_inline;
    hipStream_t st = (hipStream_t)stream;
    DeviceScope scope(device);
    if (scope.err != hipSuccess) return (int)scope.err;
    int rc = fill_params(plan, ST_Q, tensors, table, pointers, packed, packed_bytes, st, &kp, &inl, &use_inline);
    if (rc) return rc;
    if (kp.nwg == 0) return 0;
    switch (plan->dtype) {
    case TFTQ_F32: return launch_q<float>(kp, inl, use_inline, plan->wide[ST_Q], plan->parked, st);
    case TFTQ_F16: return launch_q<f16_tag>(kp, inl, use_inline, plan->wide[ST_Q], plan->parked, st);
    case TFTQ_BF16: return launch_q<bf16_tag>(kp, inl, use_inline, plan->wide[ST_Q], plan->parked, st);
    default: return TFTQ_E_DTYPE;
    }
}
