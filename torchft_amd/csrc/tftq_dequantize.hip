// k_dequantize and tftq_dequantize: fused_dequantize_from_fp8 on gfx950.
//
// Follows torchft/quantization.py:165-258 (kernel) and :591-635 (launcher); design notes in tftq_device.h.

#include "tftq_device.h"

// ---------------------------------------------------------------------------
// dequantize
// ---------------------------------------------------------------------------
// Every store of dequantized values is a streaming (nontemporal) store.  Plain stores leave
// their lines dirty in the memory-side cache, and whatever kernel runs next pays for the
// write-back (a reduce launch behind a 436 MB dequantize with plain stores: 54-58 us instead
// of 45 us, also after 200 us of idling).  Streaming stores pay off only when the pieces a
// store instruction writes are whole 64-byte blocks: partial blocks written that way are not
// merged in L2 (2000-byte bf16 rows written straight from the registers: 3.5 TB/s).  Rows that
// do not start and end on 64-byte boundaries therefore go through LDS where they can
// (dequantize_vec_rows), so that the workgroup writes whole 128-byte lines.
// True when the rows of the tensor start and end on 64-byte boundaries.
template <typename T>
DEV bool rows_fill_lines(const Seg &s)
{
    return ((s.ptr | (uint64_t)(s.row_stride * Elem<T>::ESZ) | (uint64_t)((int64_t)s.n * Elem<T>::ESZ)) & 63u) == 0;
}

// one element into the LDS image of a row
template <typename T>
DEV void stage_elem(LDS_AS uint8_t *srow, int col, float v)
{
    if constexpr (Elem<T>::ESZ == 4) *(LDS_AS u32 *)(srow + 4 * col) = as_u(v);
    else *(LDS_AS uint16_t *)(srow + 2 * col) = (uint16_t)(Elem<T>::pack2(v, 0.0f) & 0xFFFFu);
}

// The value that is stored: the quotient, or in the scaled variant (POST) the
// quotient as it reads back from the tensor's dtype, times post_scale: the
// caller's `tensor /= num_participants` (manager.py:450-452) without a second
// pass over the tensor.
template <typename T, bool POST>
DEV float fin(float v, const KParams &p)
{

    return POST ? Elem<T>::rounded(v) * p.post_scale : v;
}

// Any strides; also the path of rows whose scale is outside the range of the
// fast exact division (plain IEEE divide, one element per lane and step).
template <typename T, int TEAM, bool POST>
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
            Elem<T>::store(base, r0 + (int64_t)col * s.col_stride, fin<T, POST>(div_fast_signed(f, c.r, c.r_lo), p));
        }
    } else {
#pragma nounroll
        for (int col = lane; col < s.n; col += TEAM) {
            const float f = __builtin_amdgcn_cvt_f32_fp8((int)in[4 + col], 0);
            Elem<T>::store(base, r0 + (int64_t)col * s.col_stride, fin<T, POST>(f / c.s, p));
        }
    }
}

// Contiguous rows.  DV vectors per lane and step; their loads are issued together
// without a branch (lanes past the end re-read the last vector and do not store),
// and the first step's loads are on their way before the row's scale has arrived
// and been turned into division coefficients.  STAGED: the row is written to its
// place in LDS (srow) instead of global memory.
// v0, v1: the row's vectors v0 ... v1 - 1 only (a row dealt to several workgroups,
// tftq_d_row_parts); `last`: with the columns behind the last whole vector.
template <typename T, int TEAM, bool STAGED, int DV, bool POST>
DEV void dequantize_vec_k(const Seg &s, const KParams &p, int row, int lane, LDS_AS uint8_t *srow, int v0 = 0,
                          int v1 = -1, bool last = true)
{
    if (row >= s.m) return;
    GLOBAL const u32 *in = as_global<const u32>(p.packed + row_addr(s, p.slot_size, row));
    constexpr int EPV = Elem<T>::EPV;
    const int nvec = v1 < 0 ? s.n / EPV : v1;
    const float sraw = as_f(in[0]);
    u32x2 w[DV];
    auto load_step = [&](int base) {
#pragma unroll
        for (int k = 0; k < DV; k++) {
            const int idx = max(min(base + k * TEAM + lane, nvec - 1), 0);
            if constexpr (EPV == 4) {
                w[k].x = LOAD_STREAM(in + 1 + idx);
                w[k].y = 0;
            } else {
                w[k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)(in + 1 + 2 * idx));
            }
        }
    };
    load_step(v0);
    const DivCoef c = make_div(sraw);
    if (!c.fast) {  // same for all lanes of the team
        if constexpr (STAGED) {
#pragma nounroll
            for (int col = lane; col < s.n; col += TEAM) {
                const float f = __builtin_amdgcn_cvt_f32_fp8((int)((GLOBAL const uint8_t *)in)[4 + col], 0);
                stage_elem<T>(srow, col, fin<T, POST>(f / c.s, p));
            }
        } else if (v0 == 0) {  // the whole row, by the workgroup that has its first part
            dequantize_gen<T, TEAM, POST>(s, p, row, lane);
        }
        return;
    }
    GLOBAL u32x4_a2 *out = as_global<u32x4_a2>(s.ptr + (int64_t)row * s.row_stride * Elem<T>::ESZ);
    // the few columns after the last whole vector, one element per lane
    for (int col = (last ? nvec * EPV : s.n) + lane; col < s.n; col += TEAM) {
        const float f = __builtin_amdgcn_cvt_f32_fp8((int)((GLOBAL const uint8_t *)in)[4 + col], 0);
        const float v = fin<T, POST>(div_fast_signed(f, c.r, c.r_lo), p);
        if constexpr (STAGED) stage_elem<T>(srow, col, v);
        else Elem<T>::store(s.ptr, (int64_t)row * s.row_stride + col, v);
    }
    for (int base = v0;;) {
#pragma unroll
        for (int k = 0; k < DV; k++) {
            const int idx = base + k * TEAM + lane;
            float o[EPV];
            float f[4];
            unpack_fp8x4(w[k].x, f);
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = fin<T, POST>(div_fast_signed(f[e], c.r, c.r_lo), p);
            if constexpr (EPV == 8) {
                unpack_fp8x4(w[k].y, f);
#pragma unroll
                for (int e = 0; e < 4; e++) o[4 + e] = fin<T, POST>(div_fast_signed(f[e], c.r, c.r_lo), p);
            }
            if (idx < nvec) {
                if constexpr (STAGED) {
                    // (16-bit rows of an odd number of columns start at even bytes only)
                    if (Elem<T>::ESZ == 4 || ((uint32_t)(uintptr_t)srow & 3u) == 0) *(LDS_AS u32x4_a4 *)(srow + 16 * idx) = Elem<T>::pack(o);
                    else *(LDS_AS u32x4_a2 *)(srow + 16 * idx) = Elem<T>::pack(o);
                } else {
                    STORE_STREAM(Elem<T>::pack(o), out + idx);
                }
            }
        }
        base += DV * TEAM;
        if (base >= nvec) break;
        load_step(base);
    }
}

// One workgroup per row, a row of more than 16 KB that does not start and end on 64-byte
// boundaries: straight from the registers every wavefront's store would have partial blocks at
// both ends ([6656, 32770] bf16: 155 us against 126 us for 32768 columns), so the row goes
// through the LDS stage in pieces of 1024 vectors (16 KB), each written as whole lines; the
// columns behind the last whole vector travel with the last piece.
template <typename T, bool POST>
DEV void dequantize_vec_pieces(const Seg &s, const KParams &p, int row, int tid, uint8_t *stage, int v0, int v1, bool last)
{
    constexpr int EPV = Elem<T>::EPV, ESZ = Elem<T>::ESZ, DV = 4, STEP = DV * TFTQ_WG;
    if (row >= s.m) return;  // the whole workgroup
    GLOBAL const u32 *in = as_global<const u32>(p.packed + row_addr(s, p.slot_size, row));
    const int nvec = v1;  // this workgroup's vectors are v0 ... v1 - 1 of the row (see dequantize_vec_k)
    const DivCoef c = make_div(as_f(in[0]));
    if (!c.fast) {  // same for all lanes
        if (v0 == 0) dequantize_gen<T, TFTQ_WG, POST>(s, p, row, tid);
        return;
    }
    uint8_t *g_row = (uint8_t *)s.ptr + (int64_t)row * s.row_stride * ESZ;
#pragma nounroll
    for (int base = v0; base < nvec; base += STEP) {
        u32x2 w[DV];
#pragma unroll
        for (int k = 0; k < DV; k++) {
            const int idx = min(base + k * TFTQ_WG + tid, nvec - 1);
            if constexpr (EPV == 4) {
                w[k].x = LOAD_STREAM(in + 1 + idx);
                w[k].y = 0;
            } else {
                w[k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)(in + 1 + 2 * idx));
            }
        }
        uint8_t *g0 = g_row + (int64_t)base * 16;
        const int mis = (int)((uintptr_t)g0 & 127u);
        LDS_AS uint8_t *sp = (LDS_AS uint8_t *)stage + mis;
        const bool lastp = last && base + STEP >= nvec;
        int len = min(STEP, nvec - base) * 16;
        if (lastp) {  // the columns after the last whole vector, one element per lane
            for (int col = nvec * EPV + tid; col < s.n; col += TFTQ_WG) {
                const float f = __builtin_amdgcn_cvt_f32_fp8((int)((GLOBAL const uint8_t *)in)[4 + col], 0);
                stage_elem<T>(sp, col - base * EPV, fin<T, POST>(div_fast_signed(f, c.r, c.r_lo), p));
            }
            len += (s.n - nvec * EPV) * ESZ;
        }
#pragma unroll
        for (int k = 0; k < DV; k++) {
            const int idx = base + k * TFTQ_WG + tid;
            float o[EPV];
            float f[4];
            unpack_fp8x4(w[k].x, f);
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = fin<T, POST>(div_fast_signed(f[e], c.r, c.r_lo), p);
            if constexpr (EPV == 8) {
                unpack_fp8x4(w[k].y, f);
#pragma unroll
                for (int e = 0; e < 4; e++) o[4 + e] = fin<T, POST>(div_fast_signed(f[e], c.r, c.r_lo), p);
            }
            if (idx < nvec) {
                LDS_AS uint8_t *at = sp + 16 * (idx - base);
                if (ESZ == 4 || ((uint32_t)(uintptr_t)at & 3u) == 0) *(LDS_AS u32x4_a4 *)at = Elem<T>::pack(o);
                else *(LDS_AS u32x4_a2 *)at = Elem<T>::pack(o);
            }
        }
        __syncthreads();
        copy_out_span(stage, g0, len, tid);
        __syncthreads();  // before the next piece overwrites the stage
    }
}

// The 256 / TEAM rows of a workgroup.  Rows that start and end on 64-byte boundaries are
// written straight from the registers.  Other rows, when they are contiguous in memory
// (row stride = row length) and start at even bytes, make one span of bytes per workgroup, which
// is assembled in LDS and written as whole lines (copy_out_span); that needs the span to fit
// the stage, which the planner sees to for rows of up to 16 KB (pick_d_kind in tftq_plan.cpp).
// Longer rows go through the stage a piece at a time (dequantize_vec_pieces).  What is left
// (strided rows of up to 16 KB) is written from the registers, partial blocks included.
template <typename T, int TEAM, bool POST>
DEV void dequantize_vec_rows(const Seg &s, const KParams &p, int blk, int tid, uint8_t *stage)
{
    constexpr int R = TFTQ_WG / TEAM;
    const int r0 = blk * R;
    const int team = TEAM == 256 ? 0 : TEAM >= 64 ? __builtin_amdgcn_readfirstlane(tid / TEAM) : tid / TEAM;
    const int lane = tid & (TEAM - 1);
    const int64_t rowb = (int64_t)s.n * Elem<T>::ESZ;
    if constexpr (TEAM == TFTQ_WG) {
        const int nvec = s.n / Elem<T>::EPV;
        if (nvec >= TFTQ_D_PART_MIN) {  // a part of a long row (tftq_d_row_parts)
            const int parts = tftq_d_row_parts(K_VEC256, s.n, Elem<T>::ESZ);
            const int row = blk / parts, part = blk - row * parts;
            const int v0 = tftq_d_part_begin(nvec, parts, part), v1 = tftq_d_part_begin(nvec, parts, part + 1);
            const bool last = part == parts - 1;
            if (!rows_fill_lines<T>(s) && ((s.ptr | (uint64_t)(s.row_stride * Elem<T>::ESZ)) & 1u) == 0)
                dequantize_vec_pieces<T, POST>(s, p, row, tid, stage, v0, v1, last);
            else if (v1 - v0 <= 4 * TEAM) dequantize_vec_k<T, TEAM, false, 4, POST>(s, p, row, lane, nullptr, v0, v1, last);
            else dequantize_vec_k<T, TEAM, false, 8, POST>(s, p, row, lane, nullptr, v0, v1, last);
            return;
        }
    }
    // DV = vectors a lane loads per step: 8 in flight where the row has them (4 is 1.3 % slower
    // on 4096-column bf16 rows), 4 for shorter rows, whose lanes would mostly load duplicates
    const bool few = s.n / Elem<T>::EPV <= 4 * TEAM;
    // same branches for the whole workgroup
    if (!rows_fill_lines<T>(s) && s.row_stride == s.n && ((s.ptr | (uint64_t)rowb) & 1u) == 0 &&
        R * rowb + 127 <= TFTQ_D_STAGE) {
        uint8_t *g0 = (uint8_t *)s.ptr + (int64_t)r0 * rowb;
        const int mis = (int)((uintptr_t)g0 & 127u);
        const int len = min(R, s.m - r0) * (int)rowb;
        LDS_AS uint8_t *srow = (LDS_AS uint8_t *)stage + mis + team * (int)rowb;
        if (few) dequantize_vec_k<T, TEAM, true, 4, POST>(s, p, r0 + team, lane, srow);
        else dequantize_vec_k<T, TEAM, true, 8, POST>(s, p, r0 + team, lane, srow);
        __syncthreads();
        copy_out_span(stage, g0, len, tid);
        return;
    }
    if constexpr (TEAM == TFTQ_WG) {
        if (!rows_fill_lines<T>(s) && ((s.ptr | (uint64_t)(s.row_stride * Elem<T>::ESZ)) & 1u) == 0 &&
            s.n / Elem<T>::EPV >= 1024) {
            dequantize_vec_pieces<T, POST>(s, p, r0, tid, stage, 0, s.n / Elem<T>::EPV, true);
            return;
        }
    }
    if (few) dequantize_vec_k<T, TEAM, false, 4, POST>(s, p, r0 + team, lane, nullptr);
    else dequantize_vec_k<T, TEAM, false, 8, POST>(s, p, r0 + team, lane, nullptr);
}

// Rows of one column: one plain divide per row.  Any element stride: four rows
// per lane, interleaved.
template <typename T, bool POST>
DEV void dequantize_col1_strided(const Seg &s, const KParams &p, int row0, int tid)
{
    const float inv = 1.0f / (float)s.slice_rows;
    u32x2 w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int row = min(row0 + k * TFTQ_WG + tid, s.m - 1);
        w[k] = LOAD_STREAM((GLOBAL const u32x2_a4 *)as_global<const u32>(p.packed + row_addr_fast(s, p.slot_size, row, inv)));
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int row = row0 + k * TFTQ_WG + tid;
        const float f = __builtin_amdgcn_cvt_f32_fp8((int)w[k].y, 0);
        if (row < s.m) Elem<T>::store(s.ptr, (int64_t)row * s.row_stride, fin<T, POST>(f / as_f(w[k].x), p));  // no zero guard (:239)
    }
}

// Contiguous elements: a lane takes TFTQ_COL1_PAIRS_D pairs of neighbouring rows, reads the
// two packed rows of a pair with one 16-byte load and writes the two elements
// with one store (the mapping of quantize_col1).
template <typename T, bool POST>
DEV void dequantize_col1(const Seg &s, const KParams &p, int row0, int tid)
{
    if (s.row_stride != 1) {  // same for the whole workgroup
#pragma nounroll
        for (int r = 0; r < 2 * TFTQ_COL1_PAIRS_D * TFTQ_WG && row0 + r < s.m; r += 4 * TFTQ_WG)
            dequantize_col1_strided<T, POST>(s, p, row0 + r, tid);
        return;
    }
    const float inv = 1.0f / (float)s.slice_rows;
    u32x4 w[TFTQ_COL1_PAIRS_D];
#pragma unroll
    for (int k = 0; k < TFTQ_COL1_PAIRS_D; k++) {
        const int row = min(row0 + 2 * (k * TFTQ_WG + tid), s.m - 1);
        int slot = (int)((float)row * inv);  // off by at most one
        int j = row - slot * s.slice_rows;
        if (j < 0) { --slot; j += s.slice_rows; }
        if (j >= s.slice_rows) { ++slot; j -= s.slice_rows; }
        GLOBAL const u32 *src = as_global<const u32>(p.packed + (int64_t)slot * p.slot_size + s.slot_off + (int64_t)j * 8);
        if (j + 1 < s.slice_rows) {  // the next row follows in the same slot
            w[k] = LOAD_STREAM((GLOBAL const u32x4_a4 *)src);
        } else {
            const u32x2 a = LOAD_STREAM((GLOBAL const u32x2_a4 *)src);
            u32x2 b = {0x3F800000u, 0u};
            if (row + 1 < s.m)
                b = LOAD_STREAM((GLOBAL const u32x2_a4 *)as_global<const u32>(p.packed + row_addr_fast(s, p.slot_size, row + 1, inv)));
            w[k] = u32x4{a.x, a.y, b.x, b.y};
        }
    }
#pragma unroll
    for (int k = 0; k < TFTQ_COL1_PAIRS_D; k++) {
        const int row = row0 + 2 * (k * TFTQ_WG + tid);
        // no zero guard (:239)
        const float a = fin<T, POST>(__builtin_amdgcn_cvt_f32_fp8((int)w[k].y, 0) / as_f(w[k].x), p);
        const float b = fin<T, POST>(__builtin_amdgcn_cvt_f32_fp8((int)w[k].w, 0) / as_f(w[k].z), p);
        if (row + 1 < s.m) Elem<T>::store2(s.ptr, row, a, b);
        else if (row < s.m) Elem<T>::store(s.ptr, row, a);
    }
}

// K_VECS in dequantize: same shape as quantize_small, 8 vectors of codes and their
// rows' scales in flight per lane.  TAIL: the row is not a whole number of vectors; its last
// vector is moved back to end with the row (it overlaps its neighbour, both store the same
// values), so its codes start at any byte of the packed row.
// First column of vector idx of a row of n columns.
template <typename T>
DEV int small_vec_col(int idx, int n)
{
    return min(idx * Elem<T>::EPV, n - Elem<T>::EPV);
}

// The EPV codes from column `col` on of the packed row `in`.  TAIL: they start at any byte
// (gfx950 loads 4 and 8 bytes at any address).
typedef u32 u32_a1 __attribute__((aligned(1)));
typedef u32x2 u32x2_a1 __attribute__((aligned(1)));
template <typename T, bool TAIL>
DEV u32x2 load_small_codes(GLOBAL const u32 *in, int col)
{
    constexpr int EPV = Elem<T>::EPV;
    u32x2 w = {0u, 0u};
    if constexpr (!TAIL) {
        if constexpr (EPV == 4) w.x = LOAD_STREAM(in + 1 + (col >> 2));
        else w = LOAD_STREAM((GLOBAL const u32x2_a4 *)(in + 1 + (col >> 2)));
    } else {
        GLOBAL const uint8_t *q = (GLOBAL const uint8_t *)in + 4 + col;
        if constexpr (EPV == 4) w.x = LOAD_STREAM((GLOBAL const u32_a1 *)q);
        else w = LOAD_STREAM((GLOBAL const u32x2_a1 *)q);
    }
    return w;
}

// Rows RBEG * teams .. REND * teams - 1 of the workgroup's rows.  STAGED: they are
// neighbours in memory (row stride = row length) and go through the LDS stage as one span.
template <typename T, int C, bool STAGED, bool POST, int RBEG, int REND>
DEV void dequantize_small_rows(const Seg &s, const KParams &p, const SmallShape &h, const u32x2 (&w)[8 / C][C],
                               const float (&sc)[8 / C], bool fast, int row0, uint8_t *stage, int tid)
{
    constexpr int EPV = Elem<T>::EPV, ESZ = Elem<T>::ESZ;
    const int nvec = tftq_small_nvec(s.n, ESZ);
    const int rowb = s.n * ESZ;
    const int last = min(row0 + h.teams * (8 / C), s.m) - 1;
    const int first = row0 + RBEG * h.teams;
    if (first > last) return;  // same for the whole workgroup
    uint8_t *gp = (uint8_t *)s.ptr + (int64_t)first * rowb;  // used when STAGED
    const int mis = (int)((uintptr_t)gp & 127u);
#pragma unroll
    for (int r = RBEG; r < REND; r++) {
        const int row = row0 + r * h.teams + h.t;
        const DivCoef c = make_div(sc[r]);
        const uint64_t out = s.ptr + (uint64_t)((int64_t)min(row, s.m - 1) * s.row_stride * ESZ);
        LDS_AS uint8_t *srow = (LDS_AS uint8_t *)stage + mis + ((r - RBEG) * h.teams + h.t) * rowb;
#pragma unroll
        for (int k = 0; k < C; k++) {
            float f[4], g[4], o[EPV];
            unpack_fp8x4(w[r][k].x, f);
            unpack_fp8x4(w[r][k].y, g);
            if (fast) {
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = fin<T, POST>(div_fast_signed(f[e], c.r, c.r_lo), p);
                if constexpr (EPV == 8) {
#pragma unroll
                    for (int e = 0; e < 4; e++) o[4 + e] = fin<T, POST>(div_fast_signed(g[e], c.r, c.r_lo), p);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = fin<T, POST>(f[e] / sc[r], p);  // :250-252
                if constexpr (EPV == 8) {
#pragma unroll
                    for (int e = 0; e < 4; e++) o[4 + e] = fin<T, POST>(g[e] / sc[r], p);
                }
            }
            const int vec = k * h.team + h.l;
            if (row < s.m && vec < nvec) {
                const int at = small_vec_col<T>(vec, s.n) * ESZ;  // bytes from the start of the row
                if constexpr (STAGED) {
                    if (((uint32_t)(uintptr_t)(srow + at) & 3u) == 0) *(LDS_AS u32x4_a4 *)(srow + at) = Elem<T>::pack(o);
                    else *(LDS_AS u32x4_a2 *)(srow + at) = Elem<T>::pack(o);  // 16-bit rows of an odd number of columns
                } else {
                    STORE_STREAM(Elem<T>::pack(o), as_global<u32x4_a2>(out + (uint64_t)at));
                }
            }
        }
    }
    if constexpr (STAGED) {
        __syncthreads();
        copy_out_span(stage, gp, (min(last, row0 + REND * h.teams - 1) - first + 1) * rowb, tid);
    }
}

template <typename T, int C, bool STAGED, bool TAIL, bool POST>
DEV void dequantize_small_c(const Seg &s, const KParams &p, int blk, int tid, const SmallShape &h, uint8_t *stage)
{
    constexpr int ROWS = 8 / C;  // 8 or 4
    const int nvec = tftq_small_nvec(s.n, Elem<T>::ESZ);
    const int row0 = blk * (h.teams * ROWS);
    const float inv = 1.0f / (float)s.slice_rows;

    u32x2 w[ROWS][C];
    float sc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int row = row0 + r * h.teams + h.t;
        GLOBAL const u32 *in = as_global<const u32>(p.packed + row_addr_fast(s, p.slot_size, min(row, s.m - 1), inv));
        sc[r] = as_f(in[0]);
#pragma unroll
        for (int k = 0; k < C; k++)  // a lane past the row's last vector re-reads that one and stores nothing
            w[r][k] = load_small_codes<T, TAIL>(in, small_vec_col<T>(min(k * h.team + h.l, nvec - 1), s.n));
    }
    bool all_fast = true;
#pragma unroll
    for (int r = 0; r < ROWS; r++) all_fast = all_fast && scale_is_fast(sc[r]);
    const bool fast = __builtin_amdgcn_ballot_w64(!all_fast) == 0;  // one code path per wavefront
    // a workgroup writes up to 32 KB: two halves through the stage
    dequantize_small_rows<T, C, STAGED, POST, 0, ROWS / 2>(s, p, h, w, sc, fast, row0, stage, tid);
    if constexpr (STAGED) __syncthreads();  // the first half has been copied out of the stage
    dequantize_small_rows<T, C, STAGED, POST, ROWS / 2, ROWS>(s, p, h, w, sc, fast, row0, stage, tid);
}

template <typename T, bool STAGED, bool TAIL, bool POST>
DEV void dequantize_small_s(const Seg &s, const KParams &p, int blk, int tid, const SmallShape &h, uint8_t *stage)
{
    // one or two vectors per lane (tftq_small_shape)
    if (h.c == 1) dequantize_small_c<T, 1, STAGED, TAIL, POST>(s, p, blk, tid, h, stage);
    else dequantize_small_c<T, 2, STAGED, TAIL, POST>(s, p, blk, tid, h, stage);
}

template <typename T, bool POST>
DEV void dequantize_small(const Seg &s, const KParams &p, int blk, int tid, uint8_t *stage)
{
    const SmallShape h = small_shape(tftq_small_nvec(s.n, Elem<T>::ESZ), tid, ST_D);
    const int rowb = s.n * Elem<T>::ESZ;
    // same branches for the whole workgroup
    const bool staged = !rows_fill_lines<T>(s) && s.row_stride == s.n && ((s.ptr | (uint64_t)rowb) & 1u) == 0;
    if (s.n % Elem<T>::EPV) {
        if (staged) dequantize_small_s<T, true, true, POST>(s, p, blk, tid, h, stage);
        else dequantize_small_s<T, false, true, POST>(s, p, blk, tid, h, stage);
    } else {
        if (staged) dequantize_small_s<T, true, false, POST>(s, p, blk, tid, h, stage);
        else dequantize_small_s<T, false, false, POST>(s, p, blk, tid, h, stage);
    }
}

template <typename T, bool INLINE, bool POST>
__global__ __launch_bounds__(TFTQ_WG) void k_dequantize(const KParams p, const InlineTable inl)
{
    __shared__ __align__(16) uint8_t stage[TFTQ_D_STAGE];  // see copy_out_span
    Seg s;
    int vb;
    if (!locate<INLINE, ST_D>(p, inl, s, vb)) return;
    const int blk = vb - s.wg_begin[ST_D];
    const int tid = threadIdx.x;
    switch (s.kind[ST_D]) {
    case K_VEC256: dequantize_vec_rows<T, 256, POST>(s, p, blk, tid, stage); break;
    case K_VEC128: dequantize_vec_rows<T, 128, POST>(s, p, blk, tid, stage); break;
    case K_VEC64: dequantize_vec_rows<T, 64, POST>(s, p, blk, tid, stage); break;
    case K_VEC32: dequantize_vec_rows<T, 32, POST>(s, p, blk, tid, stage); break;
    case K_VEC16: dequantize_vec_rows<T, 16, POST>(s, p, blk, tid, stage); break;
    case K_VEC8: dequantize_vec_rows<T, 8, POST>(s, p, blk, tid, stage); break;
    case K_GEN64:
        dequantize_gen<T, 64, POST>(s, p, blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6), tid & 63);
        break;
    case K_GEN8: dequantize_gen<T, 8, POST>(s, p, blk * 32 + (tid >> 3), tid & 7); break;
    case K_GEN1: dequantize_gen<T, 1, POST>(s, p, blk * 256 + tid, 0); break;
    case K_COL1:
        if (s.m > 0) dequantize_col1<T, POST>(s, p, blk * tftq_col1_rows_per_wg(ST_D), tid);
        break;
    case K_VECS: dequantize_small<T, POST>(s, p, blk, tid, stage); break;
    default: break;
    }
}

template <typename T, bool POST>
static int launch_d(const KParams &kp, const InlineTable &inl, bool use_inline, hipStream_t st)
{
    if (use_inline) return launch_kernel(k_dequantize<T, true, POST>, grid_of(kp), 0, st, kp, inl);
    return launch_kernel(k_dequantize<T, false, POST>, grid_of(kp), 0, st, kp, inl);
}

template <bool POST>
static int dequantize(const tftq_plan *plan, void *const *tensors, const void *table, void *pointers,
                      const void *packed, int64_t packed_bytes, float post_scale, int device, void *stream)
{
    KParams kp;
    InlineTable inl = {};
    bool use_inline;
    hipStream_t st = (hipStream_t)stream;
    DeviceScope scope(device);
    if (scope.err != hipSuccess) return (int)scope.err;
    int rc = fill_params(plan, ST_D, (const void *const *)tensors, table, pointers, (void *)packed, packed_bytes, st,
                         &kp, &inl, &use_inline);
    if (rc) return rc;
    kp.post_scale = post_scale;
    if (kp.nwg == 0) return 0;
    switch (plan->dtype) {
    case TFTQ_F32: return launch_d<float, POST>(kp, inl, use_inline, st);
    case TFTQ_F16: return launch_d<f16_tag, POST>(kp, inl, use_inline, st);
    case TFTQ_BF16: return launch_d<bf16_tag, POST>(kp, inl, use_inline, st);
    default: return TFTQ_E_DTYPE;
    }
}

extern "C" int tftq_dequantize(const tftq_plan *plan, void *const *tensors, const void *table, void *pointers,
                               const void *packed, int64_t packed_bytes, int device, void *stream)
{
    return dequantize<false>(plan, tensors, table, pointers, packed, packed_bytes, 1.0f, device, stream);
}

extern "C" int tftq_dequantize_scaled(const tftq_plan *plan, void *const *tensors, const void *table,
                                      void *pointers, const void *packed, int64_t packed_bytes,
                                      float post_scale, int device, void *stream)
{
    return dequantize<true>(plan, tensors, table, pointers, packed, packed_bytes, post_scale, device, stream);
}
