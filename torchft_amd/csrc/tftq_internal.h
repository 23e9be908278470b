// Shared between the host-side planner (tftq_plan.cpp) and the HIP kernels
// (tftq_device.h and the three .hip files).  Not part of the public ABI.
#pragma once

#include <stdint.h>

#include <vector>

#include "../../include/tftq.h"

// Stages of the path, used to index per-stage fields of a segment.
enum : int { ST_Q = 0, ST_R = 1, ST_D = 2 };

// How the rows of one tensor are mapped onto lanes.  "Team" = the lanes that
// cooperate on one row.  VEC kinds (quantize, dequantize) need rows that are
// contiguous in memory (column stride 1; any row stride, any element-aligned
// start, any length); GEN kinds take any strides there.  In reduce every row of
// the packed buffer is contiguous and the GEN kinds only differ in team size.
enum : uint8_t {
    K_NONE = 0,
    K_VECS = 13,   // rows of 1-32 16-byte vectors (the last one moved back to end with the row): 1 to 32 lanes per row, several rows per lane
    K_VEC8 = 1,    // 8 lanes per row, 32 rows per workgroup
    K_VEC16 = 11,  // 16 lanes per row, 16 rows per workgroup
    K_VEC32 = 12,  // 32 lanes per row, 8 rows per workgroup
    K_VEC64 = 2,   // one wavefront per row, 4 rows per workgroup
    K_VEC128 = 14, // two wavefronts per row, 2 rows per workgroup (dequantize only)
    K_VEC256 = 3,  // one workgroup per row (also loops over rows too long for registers)
    K_GEN1 = 4,    // one lane per row, 256 rows per workgroup
    K_GEN2 = 16,   // 2 lanes per row (reduce only)
    K_GEN4 = 15,   // 4 lanes per row (reduce only)
    K_GEN8 = 5,    // 8 lanes per row
    K_GEN16 = 9,   // 16 lanes per row (reduce only)
    K_GEN32 = 10,  // 32 lanes per row (reduce only)
    K_GEN64 = 6,   // one wavefront per row
    K_GEN256 = 7,  // one workgroup per row (reduce only)
    K_COL1 = 8,    // rows of a single column (1-D tensors): 4 rows per lane, 1024 per workgroup
};

// Helpers shared by the planner (host compiler) and the kernels (hipcc).
#ifdef __HIPCC__
#define TFTQ_HD __host__ __device__
#else
#define TFTQ_HD
#endif

TFTQ_HD static inline int tftq_team_of(uint8_t kind)
{
    switch (kind) {
    case K_GEN2: return 2;
    case K_GEN4: return 4;
    case K_VEC8: case K_GEN8: return 8;
    case K_GEN16: case K_VEC16: return 16;
    case K_GEN32: case K_VEC32: return 32;
    case K_VEC64: case K_GEN64: return 64;
    case K_VEC128: return 128;
    case K_VEC256: case K_GEN256: return 256;
    case K_GEN1: return 1;
    default: return 256;
    }
}

constexpr int TFTQ_WG = 256;       // threads per workgroup, all kernels

// Reduce, teams of 64 or 256 lanes: a lane has 8 loads of 16 bytes in flight
// when the group has 8 peers.  With fewer peers a team works on 2 or 4
// consecutive rows at once so that it still has (ws = 2: 2 -> 8 loads per lane).
TFTQ_HD static inline int tftq_reduce_rows_at_once(uint8_t kind, int ndw, int ws)
{
    if (kind != K_GEN256 && kind != K_GEN64) return 1;
    const int unit_dw = tftq_team_of(kind) * 4;  // dwords that one vector per lane covers
    const int units = (ndw + unit_dw - 1) / unit_dw;  // vectors per lane and peer
    if (units == 1) return ws <= 2 ? 4 : ws <= 4 ? 2 : 1;
    if (units == 2) return ws <= 2 ? 2 : 1;
    return 1;
}

// K_VECS: a row of nvec (1..32) 16-byte vectors is owned by a team of 2^lt lanes (the
// smallest of 1, 2, 4, 8, 16 that holds it with one vector per lane; 16 lanes with two
// vectors each for 17 to 24 vectors, 32 lanes for 25 to 32), every lane holds c (1 or 2)
// vectors of it and works on 8 / c rows at once, so that it has 8 loads in flight whatever
// the row length.  A team's loads and stores should cover long runs of memory: with at most
// 8 lanes per row and up to 4 vectors per lane, 256 bf16 columns dequantized in 133.6 us
// (16 lanes of 2: 125.7 us, 32 of 1: 120.4 us), 200 columns in 154.8 us (129.6 us), 100 fp32
// columns in 239.3 us (220.0 us); quantize: 200 bf16 columns 128.9 -> 117.0 us, 136 columns
// 125.3 -> 117.3 us, 100 fp32 columns 204.9 -> 188.4 us.  (17 vectors with 32 lanes: 139.0
// against 136.5 us with 16 lanes of two.)
TFTQ_HD static inline void tftq_small_shape(int nvec, int *lt, int *c, int stage = ST_Q)
{
    (void)stage;  // quantize and dequantize take the same teams
    const int max_lt = nvec >= 25 ? 5 : 4;
    int t = 0;
    while (t < max_lt && (1 << t) < nvec) t++;
    *lt = t;
    *c = (nvec + (1 << t) - 1) >> t;
}
// vectors of a K_VECS row of n elements of esz bytes: whole ones, and one more that is moved
// back to end with the row when n is not a multiple of the vector
TFTQ_HD static inline int tftq_small_nvec(int n, int esz)
{
    const int epv = 16 / esz;
    return (n + epv - 1) / epv;
}
static inline int tftq_small_rows_per_wg(int nvec, int stage)
{
    int lt, c;
    tftq_small_shape(nvec, &lt, &c, stage);
    return (TFTQ_WG >> lt) * (8 / c);
}

// K_COL1, rows of one column.  Quantize and dequantize: a lane takes a few pairs of
// neighbouring rows and issues all its loads together.  Measured on 64 Mi rows,
// 2 / 4 / 8 pairs per lane: quantize bf16 158 / 143 / 147 us (with 2 pairs a workgroup
// has only 2 KB of input in flight and waits for it), fp32 137 / 136 / 155 us;
// dequantize bf16 118 / 117 / 122 us, fp32 131 / 140 / 147 us.
// Reduce: four rows per lane and peer.
constexpr int TFTQ_COL1_PAIRS_Q = 4, TFTQ_COL1_PAIRS_D = 2;
TFTQ_HD static inline int tftq_col1_rows_per_wg(int stage)
{
    return stage == ST_Q ? 2 * TFTQ_COL1_PAIRS_Q * TFTQ_WG
         : stage == ST_D ? 2 * TFTQ_COL1_PAIRS_D * TFTQ_WG
                         : 4 * TFTQ_WG;
}

// TFTQ_N_INLINE (tftq.h): segments that travel in the kernel arguments

// Rows a workgroup can hold in registers.  The regular kernels keep up to 8
// input vectors per lane in quantize (rows of 2048 vectors = 32 KB) and the
// accumulators of 4096 payload dwords (16384 columns) in reduce; the "wide"
// kernel variants hold twice that at half the occupancy, the wide quantize kernel
// parks another 15 vectors per lane in LDS (rows of up to 7936 vectors = 124 KB:
// 63488 bf16 or 31744 fp32 columns), and they are launched only for plans that
// contain such rows.  What a row has beyond that is read twice.
constexpr int TFTQ_Q_VECS = 8 * TFTQ_WG, TFTQ_Q_VECS_WIDE = 16 * TFTQ_WG;
constexpr int TFTQ_Q_PARKED = 15;  // more vectors per lane that the wide quantize kernel parks in LDS (60 KB)
constexpr int TFTQ_Q_PARK_GROUP = 5;  // they travel in groups of five; a row parks only the groups it needs
// groups that a row of nvec vectors parks
TFTQ_HD static inline int tftq_q_park_groups(int nvec)
{
    const int g = (nvec - TFTQ_Q_VECS_WIDE + TFTQ_Q_PARK_GROUP * TFTQ_WG - 1) / (TFTQ_Q_PARK_GROUP * TFTQ_WG);
    return g < 0 ? 0 : g > TFTQ_Q_PARKED / TFTQ_Q_PARK_GROUP ? TFTQ_Q_PARKED / TFTQ_Q_PARK_GROUP : g;
}
constexpr int TFTQ_Q_VECS_LDS = TFTQ_Q_VECS_WIDE + TFTQ_Q_PARKED * TFTQ_WG;
constexpr int TFTQ_R_DWORDS = 4096, TFTQ_R_DWORDS_WIDE = 8192;
// Dequantize assembles rows that do not fill their 64-byte blocks in LDS, one span of bytes
// per workgroup, at the offset the span has in its first 128-byte line: 16 KB + 127 bytes,
// rounded up, which leaves a CU all its workgroups.
constexpr int TFTQ_D_STAGE = 16640;

// One tensor of the list.  64 bytes.
struct Seg {
    uint64_t ptr;        // device address of element (0,0): 0 in the plan and in the table image, set per call
    int64_t slot_off;    // byte offset of this tensor's rows inside every slot
    int64_t row_stride;  // elements
    int64_t col_stride;  // elements
    int32_t m;           // real rows
    int32_t n;           // columns
    int32_t slice_rows;  // rows per slot = ceil(m / ws)
    int32_t row_bytes;   // 4 + round_up(n, 4)
    int32_t wg_begin[3]; // first workgroup of this segment, per stage
    uint8_t kind[3];     // lane mapping, per stage
    uint8_t reserved;
};
static_assert(sizeof(Seg) == 64, "Seg must be 64 bytes");

// Rows of segment s that one workgroup takes in a stage.
static inline int tftq_rows_per_wg(const Seg &s, int st, int esz, int ws)
{
    if (s.kind[st] == K_COL1) return tftq_col1_rows_per_wg(st);
    if (s.kind[st] == K_VECS) return tftq_small_rows_per_wg(tftq_small_nvec(s.n, esz), st);
    const int teams = TFTQ_WG / tftq_team_of(s.kind[st]);
    if (st == ST_R) return teams * tftq_reduce_rows_at_once(s.kind[st], s.row_bytes / 4 - 1, ws);
    return teams;
}

// Dequantize has no step that spans a row (the scale is there before the kernel starts), so
// a row of the 256-lane kind of 1536 vectors or more is dealt to several workgroups, part
// after part, four vectors per lane or fewer each: part k of a row of nvec vectors starts at
// vector floor(k * nvec / parts), rounded down to a multiple of four (64 bytes), none is
// empty, and the last one takes the columns behind the last whole vector.  [7607, 28672]
// bf16: 127.9 us with one workgroup per row, 116.1 us in parts of up to 2048 vectors.
constexpr int TFTQ_D_PART_VECS = 4 * TFTQ_WG, TFTQ_D_PART_MIN = 6 * TFTQ_WG;
TFTQ_HD static inline int tftq_d_row_parts(uint8_t kind, int n, int esz)
{
    const int nvec = n / (16 / esz);
    return kind == K_VEC256 && nvec >= TFTQ_D_PART_MIN ? (nvec + TFTQ_D_PART_VECS - 1) / TFTQ_D_PART_VECS : 1;
}
TFTQ_HD static inline int tftq_d_part_begin(int nvec, int parts, int part)
{
    return part >= parts ? nvec : (int)(((int64_t)part * nvec / parts) & ~(int64_t)3);
}
// Workgroups (or, in reduce on long lists, the workgroups that tftq_reduce_pieces turns into
// pieces) of a segment with `rows` rows in a stage.
static inline int64_t tftq_wgs_of(const Seg &s, int st, int esz, int ws, int64_t rows)
{
    const int per_wg = tftq_rows_per_wg(s, st, esz, ws);
    const int64_t wgs = (rows + per_wg - 1) / per_wg;
    return st == ST_D ? wgs * tftq_d_row_parts(s.kind[ST_D], s.n, esz) : wgs;
}

// Reduce on long lists (device table) numbers its work in quarters of workgroups, one
// wavefront each, because most tensors of such lists have a row or two per slot and a
// workgroup per tensor would be three quarters idle: wavefront w of workgroup v takes piece
// 4 v + w, finds its tensor itself, and acts as wavefront (piece - first piece) % 4 of
// workgroup (piece - first piece) / 4 of that tensor.  The kinds whose teams are wavefronts
// or less need as many pieces as have rows; the 256-lane kind, whose wavefronts meet at
// barriers, and rows of one column (rows dealt across the whole workgroup) take four pieces
// per workgroup, the former starting at a multiple of four.
static inline bool tftq_reduce_kind_has_barriers(uint8_t kind) { return kind == K_GEN256; }
static inline int64_t tftq_reduce_pieces(const Seg &s, int esz, int ws, int64_t wgs)
{
    if (wgs == 0) return 0;
    if (s.kind[ST_R] == K_GEN256 || s.kind[ST_R] == K_COL1) return 4 * wgs;
    const int per_piece = tftq_rows_per_wg(s, ST_R, esz, ws) / 4;
    return ((int64_t)s.slice_rows + per_piece - 1) / per_piece;
}


struct InlineTable {
    Seg s[TFTQ_N_INLINE];
};

// Inline tables (at most TFTQ_N_INLINE segments): XCD x works through the
// segments in the stage's work order (reduce: heaviest workgroups first;
// quantize and dequantize: list order) and takes a contiguous eighth of each.
// Its i-th piece of work belongs to the first position k with
// i < cum_end[x][k] and is workgroup base[x][k] + i of segment seg[x][k].
// Position nseg (if there is one) has seg = -1.
struct Dealt {
    int32_t cum_end[8][TFTQ_N_INLINE];  // INT32_MAX from position nseg on
    int32_t base[8][TFTQ_N_INLINE];
    int32_t seg[8][TFTQ_N_INLINE];
};

// Device tables (longer lists).  Per stage, workgroup numbers are handed out to
// the segments in the stage's work order; chunks of 2^chunk_shift consecutive
// workgroups go to the XCDs in turn, so all XCDs work down the same list.  A chunk is about 1/64 of an XCD's work and at
// least 16 workgroups: large enough that an XCD touches only its own pages of a
// big tensor, small enough that the XCDs finish together.  The device table holds
//   Seg      segs[nseg]                    in list order
//   SortEnt  sorted[3][nseg]               per stage, in workgroup order
//   MapEnt   map[3][...]                   per stage: bucket of 2^shift workgroups -> position
// and a workgroup finds its segment with one load of map[b], map[b+1] and, only
// if those differ, a binary search of sorted[] between the two positions.
struct SortEnt { int32_t begin, seg; };  // first workgroup of the segment, index into segs[]
struct MapEnt { int32_t pos, seg; };     // position in sorted[] that holds workgroup b << shift
struct TableIndex {
    int64_t sorted_off;  // bytes from the start of the device table
    int64_t map_off;
    int32_t shift;
    int32_t chunk_shift;
    int32_t per_xcd;     // workgroup ids per XCD in the grid
    int32_t pieces;      // reduce: the work is numbered in quarters of workgroups (see tftq_reduce_pieces); else 0
};

struct tftq_plan {
    int dtype;
    int esz;
    int ws;
    int nseg;
    int64_t slot_size;
    int64_t output_size;
    int64_t max_rows;
    int32_t nwg[3];
    bool wide[3];              // per stage: some row needs the kernel variant with more registers
    bool reduce_long_rows;     // every row of the list runs in a team of 64 or 256 lanes in reduce or has one column (k_reduce's R_LONG)
    int parked;                // quantize: groups of 5 vectors per lane (20 KB of LDS each, up to 3) that the longest row parks in LDS (rows above TFTQ_Q_VECS_WIDE)
    Dealt dealt[3];            // inline table only
    int32_t dealt_per_xcd[3];  // inline table only: workgroups of the busiest XCD
    bool natural[3];           // inline table only: workgroup ids keep their order (see deal_to_xcds)
    TableIndex index[3];       // device table only
    std::vector<Seg> segs;
    std::vector<uint8_t> blob;  // host image of the device table (nseg > TFTQ_N_INLINE)
};

// Kernel parameters common to the three stages.
struct KParams {
    const Seg *table;   // device table, or nullptr when the inline table is used
    const uint64_t *ptrs;  // device table only: the tensors' addresses, in list order (null in reduce)
    uint8_t *packed;
    int64_t slot_size;
    int32_t nseg;
    int32_t nwg;
    int32_t ws;
    int32_t rank;
    int32_t per_xcd;    // workgroup ids per XCD in the grid
    int32_t natural;    // inline table only: workgroup id b is piece b of the work, not piece b / 8 of XCD b % 8
    int32_t pieces;     // device table, reduce: number of quarter-workgroup pieces (0: whole workgroups)
    int32_t map_shift;  // device table only, as are the next three
    int32_t chunk_shift;
    int64_t sorted_off;
    int64_t map_off;
    Dealt dealt;        // inline table only
    int32_t div_mode;   // reduce: 0 = SUM, 1 = AVG with power-of-two ws, 2 = AVG, other ws < 1024, 3 = AVG, larger ws
    float div;          // reduce: 1.0 or float(ws)
    float inv_div;      // reduce: RN(1 / div); exact when div_mode == 1
    float post_scale;   // dequantize: factor applied to the rounded result (scaled variant only)
};
