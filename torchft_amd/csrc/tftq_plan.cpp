// Host-side planner: layout arithmetic of the packed buffer and the partition
// of rows into workgroups.  No HIP calls; compiles with any C++17 compiler.
//
// The layout restates _prepare_quantize_fp8 (torchft/quantization.py:486-503)
// and the row addressing of the kernels (:108-123).  Offsets are 64-bit here;
// the reference keeps them in int32 (:514-515).

#include <limits.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <new>
#include <vector>

#include "../../include/tftq.h"
#include "tftq_internal.h"

static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

extern "C" int tftq_version(void) { return TFTQ_VERSION; }

#ifndef TFTQ_BUILD_ID
#define TFTQ_BUILD_ID "unknown"
#endif
extern "C" const char *tftq_build_id(void) { return TFTQ_BUILD_ID; }

extern "C" const char *tftq_strerror(int code)
{
    switch (code) {
    case 0: return "success";
    case TFTQ_E_ARG: return "invalid argument";
    case TFTQ_E_DTYPE: return "Only fp32, fp16 and bf16 are supported";
    case TFTQ_E_SHAPE: return "tensor dimension out of range";
    case TFTQ_E_SIZE: return "Output size does not match";
    case TFTQ_E_NOMEM: return "out of host memory";
    case TFTQ_E_NOTABLE: return "a list of more than 16 tensors needs the device table and the pointer buffer";
    case TFTQ_E_ARCH: return "device is not gfx950";
    case TFTQ_E_TOOBIG: return "the list's descriptor table does not fit the library's fixed array";
    case TFTQ_E_BUSY: return "the library's fixed array is still in use by a call on another stream";
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
    const bool vec_ok = s.col_stride == 1 && in_bytes >= 64;
    if (s.n == 1) return K_COL1;
    const int epv = 16 / esz;
    if (s.col_stride == 1 && s.n >= epv && tftq_small_nvec(s.n, esz) <= 32)
        return K_VECS;  // short rows of at least one vector
    if (vec_ok) {
        // Team sizes measured on MI355X inside quantize -> reduce -> dequantize sequences (a
        // kernel's time depends on what ran before it, so loops over one kernel mislead):
        // 528-byte rows are fastest with 16 lanes, 1 to 4 KB rows with 32 (1000-column bf16
        // rows: 303 us per sequence against 346 us with 16 lanes), longer ones with 64.
        if (in_bytes <= 512) return K_VEC8;
        if (in_bytes <= 1024) return K_VEC16;
        if (in_bytes <= 4096) return K_VEC32;
        if (in_bytes <= 8192) return K_VEC64;
        return K_VEC256;  // longer than 32 KB: two passes inside the workgroup
    }
    if (s.n <= 16) return K_GEN1;
    if (s.n <= 128) return K_GEN8;
    return K_GEN64;
}

// Dequantize writes rows that do not start and end on 64-byte boundaries through LDS, one
// span of 256 / team rows per workgroup (dequantize_vec_rows); the team is then the largest
// whose rows fit the stage together.  Rows of more than 16 KB have few partial lines
// and keep the team of pick_io_kind, as do rows that fill their lines.
static uint8_t pick_d_kind(const Seg &s, int esz)
{
    const uint8_t k = pick_io_kind(s, esz);
    const int64_t rowb = (int64_t)s.n * esz;
    if (k != K_VEC8 && k != K_VEC16 && k != K_VEC32 && k != K_VEC64 && k != K_VEC256) return k;
    if (s.row_stride != s.n || (rowb & 63) == 0 || rowb > 16384) {
        // Written from the registers: about three to six vectors per lane (more lanes with fewer
        // vectors each cover longer runs of memory per instruction; below three the lanes have
        // too little in flight).  8 KB rows: 116.3 us with 64 lanes of 8 vectors, 110.8 us with
        // 128 of 4; 4 KB: 117.3 -> 111.3 us; 3 KB: 118.5 -> 110.9 us; 5 KB as 128 x 2.5: 105.5
        // against 102.3 us with 64 x 5; 2 KB as 64 x 2: 115.7 against 114.3 us with 32 x 4.
        // (10 KB rows: 111.9 us with 256 lanes of 2.5 vectors, 115.7 us with 128 of 5.)
        const int64_t nvec = rowb / 16;
        if (nvec > 512) return K_VEC256;
        if (nvec >= 384) return K_VEC128;
        if (nvec >= 192) return K_VEC64;
        return k;
    }
    if (rowb <= 512) return K_VEC8;
    if (rowb <= 1024) return K_VEC16;
    if (rowb <= 2048) return K_VEC32;
    if (rowb <= 4096) return K_VEC64;
    if (rowb <= 8192) return K_VEC128;
    return K_VEC256;
}

static uint8_t pick_reduce_kind(const Seg &s, int ws)
{
    // one or two 16-byte vectors of codes per lane and peer, four for the longest rows
    const int ndw = s.row_bytes / 4 - 1;
    if (s.n == 1) return K_COL1;
    // 17 to 64 bytes of codes.  A lane per row loads its row with two or four 16-byte loads that
    // lie a row apart from its neighbours'; a pair of lanes (up to 32 bytes) or a team of 4 with
    // one vector each covers 32 or 16 neighbouring rows with one load per wavefront and peer
    // and has every load of its row in flight at once (groups of up to 16 peers).  218 M bf16
    // elements, 8 peers, a lane per row against the team: 24 columns 81.1 -> 66.7 us, 28: 89.2
    // -> 64.4, 32: 65.0 -> 64.4, 44: 92.1 -> 68.7, 60: 95.6 -> 64.7, 64: 70.6 -> 65.0; 48 columns
    // (three whole vectors: a lane per row wastes nothing, the team idles a lane) 67.3 -> 69.4.
    if (ndw > 8 && ndw <= 16 && ndw != 12 && ws <= 16) return K_GEN4;
    if (ndw > 4 && ndw <= 8 && ws <= 16) return K_GEN2;
    if (ndw <= 16) return K_GEN1;  // a lane per row beats a team with idle lanes
    if (ndw <= 32) return K_GEN8;
    if (ndw <= 64) return K_GEN16;
    // Rows that would leave more than a quarter of the next team idle take three vectors per
    // lane in a team a quarter the size (the fast path of a team holds a peer's division
    // coefficients in a lane each: ws <= lanes).  2560 bf16 columns, 8 peers: 58.9 -> 48.1 us,
    // 3072: 51.6 -> 47.9, 1280: 54.2 -> 49.9, 640: 59.1 -> 53.3.  (Not below 16 lanes: 8 lanes
    // with three vectors each are slower than 32 with one, 384 columns: 62.5 against 55.5 us.)
    // (Only for tensors with rows enough to keep the machine busy: a tensor of a few rows is
    // done sooner with more lanes per row; 10 000 tensors of up to 4096 elements: 65.0 us
    // with the smaller teams, 62.8 us without.)
    const bool many = s.slice_rows >= 512;
    if (ndw <= 128) return K_GEN32;
    if (ndw <= 192 && ws <= 16 && many) return K_GEN16;
    if (ndw <= 256) return K_GEN64;
    if (ndw <= 384 && ws <= 32 && many) return K_GEN32;
    if (ndw <= 512) return K_GEN64;
    if (ndw <= 768 && ws <= 64 && many) return K_GEN64;
    return K_GEN256;
}

// Bytes one workgroup of segment s moves in a stage.
static double wg_weight(const Seg &s, int st, int esz, int ws)
{
    double rows = (double)tftq_rows_per_wg(s, st, esz, ws);
    if (st == ST_D) rows /= tftq_d_row_parts(s.kind[ST_D], s.n, esz);
    if (st == ST_R) return rows * (double)s.row_bytes * (ws + 1);
    return rows * ((double)s.n * esz + (double)s.row_bytes);
}

// The order in which a stage works through the segments.  Reduce: by workgroup
// weight, heaviest first (equal weights keep the list order), so that the last
// workgroups to finish are light; its weights differ by orders of magnitude
// within one list.  Quantize and dequantize keep the list order: their
// workgroups are all of similar weight, and sorting them measured slower.
static void work_order(const tftq_plan *p, int st, std::vector<int32_t> &ord)
{
    std::vector<double> w((size_t)p->nseg);
    ord.resize((size_t)p->nseg);
    for (int i = 0; i < p->nseg; i++) {
        ord[(size_t)i] = i;
        w[(size_t)i] = wg_weight(p->segs[(size_t)i], st, p->esz, p->ws);
    }
    if (st != ST_R) return;
    std::stable_sort(ord.begin(), ord.end(), [&](int32_t a, int32_t b) { return w[(size_t)a] > w[(size_t)b]; });
}

// Whether a stage hands its workgroups to the XCDs in their natural order (workgroup id b is
// piece b of the work: neighbouring pieces run on different XCDs at the same time and the
// whole chip works on one compact window of memory) instead of a contiguous eighth per XCD.
// Measured on MI355X, kernel sequences on 218 M elements: dequantize is 1 to 6 % faster in
// natural order (4096 bf16 columns 122.0 -> 117.9 us, 14336: 122.4 -> 115.7, 256: 148.0 ->
// 140.4, 4096 fp32: 101.4 -> 96.3) when the tensor rows are whole 64-byte blocks, and 5 %
// slower when they are not (1000 columns: neighbouring rows then share blocks across XCDs);
// quantize, which writes its packed rows as whole lines from LDS, gains 2 % (benchmark
// configuration 3: 114.0 -> 111.6 us); reduce does not care and keeps the eighths, which
// its heaviest-first order is built on.
static bool natural_order(const tftq_plan *p, int st)
{
    if (st == ST_R) return false;
    double whole = 0.0, all = 0.0;
    for (int i = 0; i < p->nseg; i++) {
        const Seg &s = p->segs[(size_t)i];
        const double bytes = (double)s.m * (double)s.n * p->esz;
        const bool fills = s.n == 1 ? s.row_stride == 1
                                    : s.col_stride == 1 && ((int64_t)s.n * p->esz) % 64 == 0 &&
                                          (s.row_stride * p->esz) % 64 == 0;
        all += bytes;
        if (fills) whole += bytes;
    }
    return whole * 2.0 >= all && all > 0.0;
}

// Few segments (the table travels in the kernel arguments).  Workgroup ids are
// dealt round-robin to the 8 XCDs by the hardware; here every XCD takes a
// contiguous eighth of every segment, so all XCDs see the same mix of row
// lengths, and works through the segments in work_order().
static void deal_to_xcds(tftq_plan *p, const int32_t (*wgs)[3])
{
    for (int st = 0; st < 3; st++) {
        int32_t begin = 0;
        for (int i = 0; i < p->nseg; i++) {  // workgroup numbers in list order
            p->segs[(size_t)i].wg_begin[st] = begin;
            begin += wgs[i][st];
        }
        std::vector<int32_t> ord;
        work_order(p, st, ord);
        Dealt &d = p->dealt[st];
        int64_t busiest = 0;
        p->natural[st] = natural_order(p, st);
        for (int x = 0; x < 8; x++) {
            int64_t cum = 0;
            for (int k = 0; k < TFTQ_N_INLINE; k++) {
                if (k >= p->nseg) {
                    d.cum_end[x][k] = INT32_MAX;
                    d.base[x][k] = 0;
                    d.seg[x][k] = -1;
                    continue;
                }
                const int i = ord[(size_t)k];
                const uint64_t n = (uint64_t)wgs[i][st];
                // natural order: every row of the table covers all workgroups of every segment
                const int64_t lo = p->natural[st] ? 0 : (int64_t)((n * (uint64_t)x) >> 3);
                const int64_t hi = p->natural[st] ? (int64_t)n : (int64_t)((n * (uint64_t)(x + 1)) >> 3);
                d.base[x][k] = (int32_t)(p->segs[(size_t)i].wg_begin[st] + lo - cum);
                d.seg[x][k] = i;
                cum += hi - lo;
                d.cum_end[x][k] = (int32_t)cum;
            }
            if (cum > busiest) busiest = cum;
        }
        p->dealt_per_xcd[st] = (int32_t)(p->natural[st] ? (busiest + 7) / 8 : busiest);
    }
}

// Many segments: the image of the device table (layout in tftq_internal.h).
static int build_table(tftq_plan *p, const int32_t (*wgs)[3])
{
    const size_t nseg = (size_t)p->nseg;
    std::vector<SortEnt> sorted[3];
    std::vector<MapEnt> map[3];
    for (int st = 0; st < 3; st++) {
        std::vector<int32_t> ord;
        work_order(p, st, ord);
        sorted[st].resize(nseg);
        // Reduce numbers quarters of workgroups (tftq_reduce_pieces), the others whole workgroups.
        const bool pieces = st == ST_R;
        int64_t begin = 0;
        for (size_t k = 0; k < nseg; k++) {  // workgroup (piece) numbers in sorted order
            const int32_t i = ord[k];
            const Seg &sg = p->segs[(size_t)i];
            if (pieces && tftq_reduce_kind_has_barriers(sg.kind[st])) begin = (begin + 3) & ~(int64_t)3;
            if (begin > INT32_MAX - 4096) return TFTQ_E_SHAPE;
            p->segs[(size_t)i].wg_begin[st] = (int32_t)begin;
            sorted[st][k] = SortEnt{(int32_t)begin, i};
            begin += pieces ? tftq_reduce_pieces(sg, p->esz, p->ws, wgs[i][st]) : wgs[i][st];
        }
        if (begin > INT32_MAX - 4096) return TFTQ_E_SHAPE;
        p->index[st].pieces = pieces ? (int32_t)begin : 0;
        if (pieces) p->nwg[st] = (int32_t)((begin + 3) / 4);
        const int64_t nwg = begin;  // what the map is indexed by
        int shift = 0;
        while ((nwg >> shift) > 4 * (int64_t)nseg) shift++;
        const int64_t nb = (nwg >> shift) + 1;  // buckets; map[] has one more entry
        map[st].resize((size_t)nb + 1);
        size_t k = 0;
        for (int64_t b = 0; b <= nb; b++) {
            const int64_t w = b << shift;
            if (w >= nwg) {
                k = nseg - 1;
            } else {
                while (k + 1 < nseg && sorted[st][k + 1].begin <= w) k++;
            }
            map[st][(size_t)b] = MapEnt{(int32_t)k, sorted[st][k].seg};
        }
        p->index[st].shift = shift;
        const int64_t nwgs = p->nwg[st];  // workgroups of the launch
        int cs = 4;
        while (cs < 20 && (nwgs >> (cs + 1)) >= 8 * 64) cs++;
        p->index[st].chunk_shift = cs;
        const int64_t turns = (nwgs + ((int64_t)8 << cs) - 1) / ((int64_t)8 << cs);
        p->index[st].per_xcd = (int32_t)(turns << cs);
    }
    size_t bytes = nseg * sizeof(Seg);
    for (int st = 0; st < 3; st++) {
        p->index[st].sorted_off = (int64_t)bytes;
        bytes += nseg * sizeof(SortEnt);
    }
    for (int st = 0; st < 3; st++) {
        p->index[st].map_off = (int64_t)bytes;
        bytes += map[st].size() * sizeof(MapEnt);
    }
    p->blob.resize(bytes);
    memcpy(p->blob.data(), p->segs.data(), nseg * sizeof(Seg));
    for (int st = 0; st < 3; st++) {
        memcpy(p->blob.data() + p->index[st].sorted_off, sorted[st].data(), nseg * sizeof(SortEnt));
        memcpy(p->blob.data() + p->index[st].map_off, map[st].data(), map[st].size() * sizeof(MapEnt));
    }
    return 0;
}

extern "C" int tftq_plan_create(int dtype, int n_tensors, const int64_t *shapes, const int64_t *strides,
                                int ws, tftq_plan **out)
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
    p->max_rows = 0;
    std::vector<int64_t> offs;
    std::vector<int32_t> wgs_flat;
    try {  // nothing may throw across the C ABI
        p->segs.resize((size_t)n_tensors);
        offs.resize((size_t)n_tensors);
        wgs_flat.resize((size_t)n_tensors * 3);
    } catch (...) {
        delete p;
        return TFTQ_E_NOMEM;
    }
    int rc = tftq_layout(n_tensors, shapes, ws, offs.data(), &p->slot_size, &p->output_size);
    if (rc) {
        delete p;
        return rc;
    }
    int64_t wg[3] = {0, 0, 0};
    int32_t (*wgs)[3] = (int32_t (*)[3])wgs_flat.data();  // workgroups per segment and stage
    for (int i = 0; i < n_tensors; i++) {
        Seg &s = p->segs[(size_t)i];
        memset(&s, 0, sizeof(s));
        s.ptr = 0;
        s.slot_off = offs[(size_t)i];
        s.m = (int32_t)shapes[2 * i];
        s.n = (int32_t)shapes[2 * i + 1];
        s.row_stride = strides[2 * i];
        s.col_stride = strides[2 * i + 1];
        s.slice_rows = (int32_t)cdiv64(s.m, ws);
        s.row_bytes = (int32_t)((cdiv64(s.n, 4) + 1) * 4);
        const int64_t m_pad = (int64_t)s.slice_rows * ws;
        if (m_pad > p->max_rows) p->max_rows = m_pad;

        s.kind[ST_Q] = pick_io_kind(s, p->esz);
        s.kind[ST_D] = pick_d_kind(s, p->esz);
        s.kind[ST_R] = pick_reduce_kind(s, p->ws);
        const int64_t rows[3] = {m_pad, s.slice_rows, s.m};
        for (int st = 0; st < 3; st++) {
            const int64_t n = tftq_wgs_of(s, st, p->esz, ws, rows[st]);
            wgs[i][st] = (int32_t)n;
            wg[st] += n;
            if (wg[st] > INT32_MAX - 4096) {
                delete p;
                return TFTQ_E_SHAPE;
            }
        }
    }
    for (int st = 0; st < 3; st++) p->nwg[st] = (int32_t)wg[st];
    p->wide[ST_Q] = p->wide[ST_R] = p->wide[ST_D] = false;
    p->parked = 0;
    p->natural[ST_Q] = p->natural[ST_R] = p->natural[ST_D] = false;
    p->reduce_long_rows = true;
    for (int i = 0; i < n_tensors; i++) {
        const Seg &s = p->segs[(size_t)i];
        const int nvec = s.n / (16 / p->esz), ndw = s.row_bytes / 4 - 1;
        if (s.m > 0 && s.kind[ST_R] != K_GEN256 && s.kind[ST_R] != K_GEN64 && s.kind[ST_R] != K_COL1)
            p->reduce_long_rows = false;
        if (s.kind[ST_Q] == K_VEC256 && nvec > TFTQ_Q_VECS && s.m > 0) p->wide[ST_Q] = true;
        if (s.kind[ST_Q] == K_VEC256 && nvec > TFTQ_Q_VECS_WIDE && s.m > 0) p->parked = std::max(p->parked, tftq_q_park_groups(nvec));
        if (s.kind[ST_R] == K_GEN256 && ndw > TFTQ_R_DWORDS && s.m > 0 && ws <= 64)
            p->wide[ST_R] = true;

    }
    try {
        if (p->nseg <= TFTQ_N_INLINE) {
            deal_to_xcds(p, wgs);
        } else if (const int rc = build_table(p, wgs)) {
            delete p;
            return rc;
        }
    } catch (...) {
        delete p;
        return TFTQ_E_NOMEM;
    }
    // a grid has fewer than 2^32 threads
    for (int st = 0; st < 3; st++) {
        const int64_t per_xcd = p->nseg <= TFTQ_N_INLINE ? p->dealt_per_xcd[st] : p->index[st].per_xcd;
        if (8 * per_xcd * TFTQ_WG > (int64_t)UINT32_MAX) {
            delete p;
            return TFTQ_E_SHAPE;
        }
    }
    *out = p;
    return 0;
}

extern "C" void tftq_plan_destroy(tftq_plan *plan) { delete plan; }

extern "C" int64_t tftq_plan_output_size(const tftq_plan *plan) { return plan ? plan->output_size : -1; }
extern "C" int64_t tftq_plan_slot_size(const tftq_plan *plan) { return plan ? plan->slot_size : -1; }
extern "C" int64_t tftq_plan_max_rows(const tftq_plan *plan) { return plan ? plan->max_rows : -1; }
extern "C" int tftq_plan_n_tensors(const tftq_plan *plan) { return plan ? plan->nseg : -1; }

extern "C" int64_t tftq_plan_table_bytes(const tftq_plan *plan)
{
    if (!plan) return -1;
    return plan->nseg > TFTQ_N_INLINE ? (int64_t)plan->blob.size() : 0;
}

extern "C" const void *tftq_plan_table_host(const tftq_plan *plan)
{
    if (!plan) return nullptr;
    return plan->nseg > TFTQ_N_INLINE ? (const void *)plan->blob.data() : nullptr;
}
