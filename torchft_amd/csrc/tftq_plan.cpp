// Host-side planner: layout arithmetic of the packed buffer and the partition
// of rows into workgroups.  No HIP calls; compiles with any C++17 compiler.
//
// The layout restates _prepare_quantize_fp8 (torchft/quantization.py:486-503)
// and the row addressing of the kernels (:108-123).  Offsets are 64-bit here;
// the reference keeps them in int32 (:514-515).

#include <limits.h>
#include <stdlib.h>
#include <string.h>

#include <new>

#include "../../include/tftq.h"
#include "tftq_internal.h"

static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

extern "C" int tftq_version(void) { return TFTQ_VERSION; }

extern "C" const char *tftq_strerror(int code)
{
    switch (code) {
    case 0: return "success";
    case TFTQ_E_ARG: return "invalid argument";
    case TFTQ_E_DTYPE: return "Only fp32, fp16 and bf16 are supported";
    case TFTQ_E_SHAPE: return "tensor dimension out of range";
    case TFTQ_E_SIZE: return "Output size does not match";
    case TFTQ_E_NOMEM: return "out of host memory";
    case TFTQ_E_NOTABLE: return "plan needs a device descriptor table";
    case TFTQ_E_ARCH: return "device is not gfx950";
    default: return code > 0 ? "HIP error" : "unknown error";
    }
}

extern "C" int tftq_layout(int n_tensors, const int64_t *shapes, int ws, int64_t *slot_off,
                           int64_t *slot_size, int64_t *output_size)
{
    if (n_tensors <= 0 || !shapes || ws <= 0) return TFTQ_E_ARG;
    int64_t per_rank = 0;
    for (int i = 0; i < n_tensors; i++) {
        const int64_t m = shapes[2 * i], n = shapes[2 * i + 1];
        if (m < 0 || n < 0 || m > INT32_MAX - ws || n > INT32_MAX - 8) return TFTQ_E_SHAPE;
        const int64_t row_bytes = (cdiv64(n, 4) + 1) * 4;
        if (slot_off) slot_off[i] = per_rank;
        per_rank += cdiv64(m, ws) * row_bytes;
        if (per_rank > (INT64_MAX / 2) / ws) return TFTQ_E_SHAPE;
    }
    if (slot_size) *slot_size = per_rank;
    if (output_size) *output_size = per_rank * ws;
    return 0;
}

static uint8_t pick_io_kind(const Seg &s, int esz)
{
    // Vector kinds: contiguous rows of at least 64 bytes.  Neither the row start nor the
    // row length needs to be a multiple of 16 bytes: gfx950 loads and stores 16-byte
    // vectors at element alignment, and a short tail is handled per element.
    const int64_t in_bytes = (int64_t)s.n * esz;
    const bool vec_ok = s.ptr != 0 && s.col_stride == 1 && in_bytes >= 64;
    if (s.n == 1 && s.ptr != 0) return K_COL1;
    if (vec_ok) {
        if (in_bytes <= 1024) return K_VEC8;
        if (in_bytes <= 8192) return K_VEC64;
        return K_VEC256;  // longer than 32 KB: two passes inside the workgroup
    }
    if (s.n <= 16) return K_GEN1;
    if (s.n <= 128) return K_GEN8;
    return K_GEN64;
}

static uint8_t pick_reduce_kind(const Seg &s)
{
    // one or two 16-byte vectors of codes per lane and peer, four for the longest rows
    const int ndw = s.row_bytes / 4 - 1;
    if (s.n == 1) return K_COL1;
    if (ndw <= 4) return K_GEN1;
    if (ndw <= 32) return K_GEN8;
    if (ndw <= 512) return K_GEN64;
    return K_GEN256;
}

// Reduce: a wide team works through several consecutive short rows, prefetching
// the next one; about 32 KB of peer rows per team (measured best on MI355X:
// more rows per team leave too few workgroups to balance the CUs).
static int reduce_team_bytes() { return 32 * 1024; }

static int pick_reduce_rows(const Seg &s, int ws)
{
    if (s.kind[ST_R] != K_GEN256 && s.kind[ST_R] != K_GEN64) return 1;
    const int64_t per_row = (int64_t)s.row_bytes * ws;
    int64_t r = (reduce_team_bytes() + per_row / 2) / per_row;
    if (r < 1) r = 1;
    if (r > 16) r = 16;
    return (int)r;
}

static int rows_per_wg_of(const Seg &s, int st)
{
    if (s.kind[st] == K_COL1) return 4 * TFTQ_WG;
    const int teams = TFTQ_WG / tftq_team_of(s.kind[st]);
    return st == ST_R ? teams * s.reduce_rows_per_team : teams;
}

// Bytes one workgroup of segment s moves in a stage.
static double wg_weight(const Seg &s, int st, int esz, int ws)
{
    const double rows = (double)rows_per_wg_of(s, st);
    if (st == ST_R) return rows * (double)s.row_bytes * (ws + 1);
    return rows * ((double)s.n * esz + (double)s.row_bytes);
}

// Workgroup ids are dealt round-robin to the 8 XCDs by the hardware; the
// kernels turn that into one contiguous range of workgroups per XCD.  Choose
// the ranges so that every XCD moves about the same number of bytes (rows of
// different tensors differ in length by up to 3.5x in one call).
static void balance_xcds(tftq_plan *p)
{
    for (int st = 0; st < 3; st++) {
        int32_t *xb = p->xcd_begin[st];
        const int nwg = p->nwg[st];
        double total = 0;
        for (int i = 0; i < p->nseg; i++) {
            const Seg &s = p->segs[(size_t)i];
            const int end = i + 1 < p->nseg ? p->segs[(size_t)i + 1].wg_begin[st] : nwg;
            total += (double)(end - s.wg_begin[st]) * wg_weight(s, st, p->esz, p->ws);
        }
        xb[0] = 0;
        int x = 1;
        double cum = 0;
        for (int i = 0; i < p->nseg && x < 8; i++) {
            const Seg &s = p->segs[(size_t)i];
            const int begin = s.wg_begin[st];
            const int end = i + 1 < p->nseg ? p->segs[(size_t)i + 1].wg_begin[st] : nwg;
            const double w = wg_weight(s, st, p->esz, p->ws);
            if (end == begin || w <= 0) continue;
            const double seg_total = (double)(end - begin) * w;
            while (x < 8 && cum + seg_total >= total * x / 8.0) {
                double k = (total * x / 8.0 - cum) / w;  // workgroups of this segment before the cut
                int cut = begin + (int)(k + 0.5);
                if (cut < xb[x - 1]) cut = xb[x - 1];
                if (cut > end) cut = end;
                xb[x++] = cut;
            }
            cum += seg_total;
        }
        while (x <= 8) xb[x++] = nwg;
        xb[8] = nwg;
    }
}

// Few segments (the table travels in the kernel arguments): every XCD takes a
// contiguous eighth of every segment, so all XCDs see the same mix of row
// lengths, and works through the segments with the heaviest workgroups first,
// so the last workgroups to finish are light ones.
static void deal_to_xcds(tftq_plan *p)
{
    if (p->nseg > TFTQ_N_INLINE) return;
    for (int st = 0; st < 3; st++) {
        uint8_t ord[TFTQ_N_INLINE];
        double w[TFTQ_N_INLINE];
        for (int i = 0; i < p->nseg; i++) {
            ord[i] = (uint8_t)i;
            w[i] = wg_weight(p->segs[(size_t)i], st, p->esz, p->ws);
        }
        for (int i = 1; i < p->nseg; i++)  // stable insertion sort, descending weight
            for (int j = i; j > 0 && w[ord[j]] > w[ord[j - 1]]; j--) {
                const uint8_t t = ord[j];
                ord[j] = ord[j - 1];
                ord[j - 1] = t;
            }
        Dealt &d = p->dealt[st];
        int64_t busiest = 0;
        for (int x = 0; x < 8; x++) {
            int64_t cum = 0;
            for (int k = 0; k < TFTQ_N_INLINE; k++) {
                if (k >= p->nseg) {
                    d.cum_end[x][k] = INT32_MAX;
                    d.base[x][k] = 0;
                    d.seg[x][k] = -1;
                    continue;
                }
                const int i = ord[k];
                const int begin = p->segs[(size_t)i].wg_begin[st];
                const int end = i + 1 < p->nseg ? p->segs[(size_t)i + 1].wg_begin[st] : p->nwg[st];
                const uint64_t wgs = (uint64_t)(end - begin);
                const int64_t lo = (int64_t)((wgs * (uint64_t)x) >> 3);
                const int64_t hi = (int64_t)((wgs * (uint64_t)(x + 1)) >> 3);
                d.base[x][k] = (int32_t)(begin + lo - cum);
                d.seg[x][k] = i;
                cum += hi - lo;
                d.cum_end[x][k] = (int32_t)cum;
            }
            if (cum > busiest) busiest = cum;
        }
        p->dealt_per_xcd[st] = (int32_t)busiest;
    }
}

extern "C" int tftq_plan_create(int dtype, int n_tensors, const void *const *ptrs,
                                const int64_t *shapes, const int64_t *strides, int ws,
                                tftq_plan **out)
{
    if (!out) return TFTQ_E_ARG;
    *out = nullptr;
    if (dtype != TFTQ_F32 && dtype != TFTQ_F16 && dtype != TFTQ_BF16) return TFTQ_E_DTYPE;
    if (n_tensors <= 0 || !shapes || !strides || ws <= 0) return TFTQ_E_ARG;

    tftq_plan *p = new (std::nothrow) tftq_plan();
    if (!p) return TFTQ_E_NOMEM;
    p->dtype = dtype;
    p->esz = dtype == TFTQ_F32 ? 4 : 2;
    p->ws = ws;
    p->nseg = n_tensors;
    p->device_table = nullptr;
    p->max_rows = 0;
    try {
        p->segs.resize((size_t)n_tensors);
    } catch (...) {
        delete p;
        return TFTQ_E_NOMEM;
    }
    std::vector<int64_t> offs((size_t)n_tensors);
    int rc = tftq_layout(n_tensors, shapes, ws, offs.data(), &p->slot_size, &p->output_size);
    if (rc) {
        delete p;
        return rc;
    }
    int64_t wg[3] = {0, 0, 0};
    for (int i = 0; i < n_tensors; i++) {
        Seg &s = p->segs[(size_t)i];
        memset(&s, 0, sizeof(s));
        s.ptr = ptrs ? (uint64_t)(uintptr_t)ptrs[i] : 0;
        s.slot_off = offs[(size_t)i];
        s.m = (int32_t)shapes[2 * i];
        s.n = (int32_t)shapes[2 * i + 1];
        s.row_stride = strides[2 * i];
        s.col_stride = strides[2 * i + 1];
        s.slice_rows = (int32_t)cdiv64(s.m, ws);
        s.row_bytes = (int32_t)((cdiv64(s.n, 4) + 1) * 4);
        const int64_t m_pad = (int64_t)s.slice_rows * ws;
        if (m_pad > p->max_rows) p->max_rows = m_pad;

        s.kind[ST_Q] = s.kind[ST_D] = pick_io_kind(s, p->esz);
        s.kind[ST_R] = pick_reduce_kind(s);
        s.reduce_rows_per_team = (uint8_t)pick_reduce_rows(s, ws);
        const int64_t rows[3] = {m_pad, s.slice_rows, s.m};
        for (int st = 0; st < 3; st++) {
            s.wg_begin[st] = (int32_t)wg[st];
            const int rows_per_wg = rows_per_wg_of(s, st);
            wg[st] += cdiv64(rows[st], rows_per_wg);
            if (wg[st] > INT32_MAX - 16) {
                delete p;
                return TFTQ_E_SHAPE;
            }
        }
    }
    for (int st = 0; st < 3; st++) p->nwg[st] = (int32_t)wg[st];
    balance_xcds(p);
    deal_to_xcds(p);
    *out = p;
    return 0;
}

extern "C" void tftq_plan_destroy(tftq_plan *plan) { delete plan; }

extern "C" int64_t tftq_plan_output_size(const tftq_plan *plan) { return plan ? plan->output_size : -1; }
extern "C" int64_t tftq_plan_slot_size(const tftq_plan *plan) { return plan ? plan->slot_size : -1; }
extern "C" int64_t tftq_plan_max_rows(const tftq_plan *plan) { return plan ? plan->max_rows : -1; }

extern "C" int64_t tftq_plan_table_bytes(const tftq_plan *plan)
{
    if (!plan) return -1;
    return plan->nseg > TFTQ_N_INLINE ? (int64_t)plan->nseg * (int64_t)sizeof(Seg) : 0;
}

extern "C" const void *tftq_plan_table_host(const tftq_plan *plan)
{
    return plan ? (const void *)plan->segs.data() : nullptr;
}

extern "C" int tftq_plan_set_device_table(tftq_plan *plan, const void *device_table)
{
    if (!plan) return TFTQ_E_ARG;
    plan->device_table = device_table;
    return 0;
}
