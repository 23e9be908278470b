// Host check of the workgroup -> (tensor, block) mapping that the kernels use.
//
// For random tensor lists this program builds plans with the library's own
// planner (tftq_plan.cpp, linked in), walks every workgroup id of the launch
// grid through a host restatement of the kernels' lookup (inline tables: the
// per-XCD dealt rows; device tables: chunk dealing, bucket map, binary search,
// and for reduce the quarters of workgroups that its wavefronts take one each)
// and checks that every block of every tensor is visited exactly once, in all
// three stages.  Prints "ok <plans> plans" on success.

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "../include/tftq.h"
#include "../torchft_amd/csrc/tftq_internal.h"

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd()
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (uint32_t)(rng_state >> 32);
}

// (segment, workgroup number) of workgroup id b, or false when b has no work
static bool locate_inline(const tftq_plan *p, int st, uint32_t b, int *seg, int *vb)
{
    const int x = (int)(b & 7), i = p->natural[st] ? (int)b : (int)(b >> 3);
    const Dealt &d = p->dealt[st];
    int base = d.base[x][0], sg = d.seg[x][0];
    for (int j = 1; j < TFTQ_N_INLINE; j++)
        if (i >= d.cum_end[x][j - 1]) {
            base = d.base[x][j];
            sg = d.seg[x][j];
        }
    if (sg < 0 || i >= d.cum_end[x][TFTQ_N_INLINE - 1]) return false;
    *seg = sg;
    *vb = base + i;
    return true;
}

// wave: the wavefront of the workgroup (stages that number quarters of workgroups: reduce)
static bool locate_table(const tftq_plan *p, int st, uint32_t b, int wave, int *seg, int *vb, size_t *max_steps)
{
    const int x = (int)(b & 7), i = (int)(b >> 3);
    const int cs = p->index[st].chunk_shift;
    int v = ((((i >> cs) << 3) + x) << cs) + (i & ((1 << cs) - 1));
    if (v >= p->nwg[st]) return false;
    if (p->index[st].pieces) {
        v = 4 * v + wave;
        if (v >= p->index[st].pieces) return false;
    }
    const uint8_t *tab = p->blob.data();
    const size_t map_idx = (size_t)(v >> p->index[st].shift);
    const size_t map_bytes = (size_t)p->index[st].map_off + (map_idx + 2) * sizeof(MapEnt);
    if (map_bytes > p->blob.size()) {
        printf("map read past the table: stage %d wg %d\n", st, v);
        exit(1);
    }
    const MapEnt *m = (const MapEnt *)(tab + p->index[st].map_off) + map_idx;
    int lo = m[0].pos, sg = m[0].seg, hi = m[1].pos;
    if (lo < 0 || hi >= p->nseg || lo > hi) {
        printf("bad map entry: stage %d wg %d lo %d hi %d\n", st, v, lo, hi);
        exit(1);
    }
    if (lo != hi) {
        const SortEnt *sorted = (const SortEnt *)(tab + p->index[st].sorted_off);
        size_t steps = 0;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (sorted[mid].begin <= v) lo = mid; else hi = mid - 1;
            steps++;
        }
        if (steps > *max_steps) *max_steps = steps;
        sg = sorted[lo].seg;
    }
    *seg = sg;
    *vb = v;
    return true;
}

static int check_plan(const std::vector<int64_t> &shapes, int ws, int dtype)
{
    const int n = (int)shapes.size() / 2;
    std::vector<int64_t> strides((size_t)n * 2);
    for (int i = 0; i < n; i++) {
        strides[2 * (size_t)i] = shapes[2 * (size_t)i + 1];
        strides[2 * (size_t)i + 1] = 1;
    }
    tftq_plan *p = nullptr;
    const int rc = tftq_plan_create(dtype, n, shapes.data(), strides.data(), ws, &p);
    if (rc) {
        printf("plan_create failed: %d\n", rc);
        return 1;
    }
    const bool inl = n <= TFTQ_N_INLINE;
    if (!inl) {  // the table image starts with the descriptors in list order
        if (p->blob.size() != (size_t)tftq_plan_table_bytes(p) || tftq_plan_table_host(p) != p->blob.data() ||
            memcmp(p->blob.data(), p->segs.data(), (size_t)n * sizeof(Seg)) != 0) {
            printf("table image mismatch\n");
            return 1;
        }
    }
    for (int st = 0; st < 3; st++) {
        // blocks each segment must receive: workgroups, or quarters of workgroups (pieces)
        const bool pieces = !inl && p->index[st].pieces > 0;
        if (pieces != (!inl && st == ST_R)) {
            printf("stage %d: pieces %d\n", st, (int)pieces);
            return 1;
        }
        std::vector<std::vector<uint8_t>> seen((size_t)n);
        int64_t total = 0;
        for (int i = 0; i < n; i++) {
            const Seg &s = p->segs[(size_t)i];
            const int64_t m_pad = (int64_t)s.slice_rows * ws;
            const int64_t rows = st == ST_Q ? m_pad : st == ST_R ? s.slice_rows : s.m;
            const int per_wg = tftq_rows_per_wg(s, st, dtype == TFTQ_F32 ? 4 : 2, ws);
            int64_t blocks = (rows + per_wg - 1) / per_wg;
            if (st == ST_D) {  // long rows of dequantize are dealt to several workgroups
                const int epv = dtype == TFTQ_F32 ? 4 : 8;
                const int nvec = s.n / epv;
                const int parts = s.kind[ST_D] == K_VEC256 && nvec >= 1536 ? (nvec + 1023) / 1024 : 1;
                bool ok = parts == tftq_d_row_parts(s.kind[ST_D], s.n, 16 / epv) && tftq_d_part_begin(nvec, parts, 0) == 0 &&
                          tftq_d_part_begin(nvec, parts, parts) == nvec;
                for (int k = 0; k < parts && ok && parts > 1; k++) {  // parts in order, none empty, none longer than a step
                    const int a = tftq_d_part_begin(nvec, parts, k), b = tftq_d_part_begin(nvec, parts, k + 1);
                    ok = a < b && b - a <= 1024 + 3 && (a & 3) == 0;
                }
                if (!ok) {
                    printf("segment %d: %d parts for %d vectors\n", i, parts, nvec);
                    return 1;
                }
                blocks *= parts;
            }
            if (pieces) {
                blocks = tftq_reduce_pieces(s, dtype == TFTQ_F32 ? 4 : 2, ws, blocks);
                // every row of the tensor lies in one of its pieces
                const bool whole = s.kind[st] == K_GEN256 || s.kind[st] == K_COL1;
                if (whole ? blocks * per_wg < 4 * rows : blocks * (per_wg / 4) < rows || (blocks - 1) * (per_wg / 4) >= rows + (rows == 0)) {
                    printf("stage %d segment %d: %lld pieces for %lld rows\n", st, i, (long long)blocks, (long long)rows);
                    return 1;
                }
                if (tftq_reduce_kind_has_barriers(s.kind[st]) && (s.wg_begin[st] & 3)) {
                    printf("stage %d segment %d: a kind with barriers starts at piece %d\n", st, i, s.wg_begin[st]);
                    return 1;
                }
            }
            seen[(size_t)i].assign((size_t)blocks, 0);
            total += blocks;
        }
        const int64_t launched = pieces ? 4 * (int64_t)p->nwg[st] : p->nwg[st];
        if (pieces ? (total > p->index[st].pieces || p->index[st].pieces > launched || launched > p->index[st].pieces + 3)
                   : total != p->nwg[st]) {
            printf("stage %d: %lld blocks but nwg %d\n", st, (long long)total, p->nwg[st]);
            return 1;
        }
        const int64_t per_xcd = inl ? p->dealt_per_xcd[st] : p->index[st].per_xcd;
        const int64_t grid = 8 * per_xcd;
        const int64_t wgs_needed = p->nwg[st];
        const int64_t slack = inl ? 8 * n : ((int64_t)8 << p->index[st].chunk_shift) + wgs_needed / 32;
        if (grid < wgs_needed || grid > wgs_needed + slack) {
            printf("stage %d: grid %lld for %lld workgroups\n", st, (long long)grid, (long long)wgs_needed);
            return 1;
        }
        int64_t visited = 0;
        size_t max_steps = 0;
        for (int64_t b = 0; b < grid; b++) {
            for (int wave = 0; wave < (pieces ? 4 : 1); wave++) {
                int sg = -1, vb = -1;
                const bool ok = inl ? locate_inline(p, st, (uint32_t)b, &sg, &vb)
                                    : locate_table(p, st, (uint32_t)b, wave, &sg, &vb, &max_steps);
                if (!ok) continue;
                if (sg < 0 || sg >= n) {
                    printf("stage %d id %lld: segment %d\n", st, (long long)b, sg);
                    return 1;
                }
                const int64_t blk = (int64_t)vb - p->segs[(size_t)sg].wg_begin[st];
                if (pieces && blk >= (int64_t)seen[(size_t)sg].size()) {
                    // padding in front of a tensor whose kind needs whole workgroups: it must
                    // fall to a kind whose wavefronts simply find no row
                    if (blk >= 0 && !tftq_reduce_kind_has_barriers(p->segs[(size_t)sg].kind[st]) && blk < (int64_t)seen[(size_t)sg].size() + 3)
                        continue;
                }
                if (blk < 0 || blk >= (int64_t)seen[(size_t)sg].size() || seen[(size_t)sg][(size_t)blk]) {
                    printf("stage %d id %lld: segment %d block %lld out of range or visited twice\n", st,
                           (long long)b, sg, (long long)blk);
                    return 1;
                }
                if (pieces && tftq_reduce_kind_has_barriers(p->segs[(size_t)sg].kind[st]) && (blk & 3) != wave) {
                    printf("stage %d id %lld: a workgroup of a kind with barriers is split\n", st, (long long)b);
                    return 1;
                }
                seen[(size_t)sg][(size_t)blk] = 1;
                visited++;
            }
        }
        if (visited != total) {
            printf("stage %d: visited %lld of %lld\n", st, (long long)visited, (long long)total);
            return 1;
        }
        if (max_steps > 16) {
            printf("stage %d: %zu search steps\n", st, max_steps);
            return 1;
        }
    }
    tftq_plan_destroy(p);
    return 0;
}

int main()
{
    int plans = 0;
    // hand-picked lists: the Llama-3-8B layer bucket, empty tensors, one huge and many tiny
    const int64_t llama[] = {4096, 4096, 1024, 4096, 1024, 4096, 4096, 4096, 14336, 4096,
                             14336, 4096, 4096, 14336, 4096, 1, 4096, 1};
    if (check_plan(std::vector<int64_t>(llama, llama + 18), 8, TFTQ_BF16)) return 1;
    plans++;
    {
        std::vector<int64_t> s;
        for (int i = 0; i < 40; i++) {
            s.push_back(i % 3 == 0 ? 0 : 7 * i);
            s.push_back(i % 5 == 0 ? 0 : 3 * i + 1);
        }
        if (check_plan(s, 4, TFTQ_F32)) return 1;
        plans++;
    }
    {
        std::vector<int64_t> s = {200000, 2048};
        for (int i = 0; i < 3000; i++) {
            s.push_back(1 + i % 7);
            s.push_back(1 + i % 33);
        }
        s.push_back(0);
        s.push_back(5);
        if (check_plan(s, 16, TFTQ_BF16)) return 1;
        plans++;
    }
    // random lists on both sides of the inline limit
    for (int it = 0; it < 300; it++) {
        const int n = 1 + (int)(rnd() % (it % 3 == 0 ? 16 : it % 3 == 1 ? 64 : 700));
        const int ws = 1 + (int)(rnd() % 17);
        std::vector<int64_t> s;
        for (int i = 0; i < n; i++) {
            const uint32_t kind = rnd() % 8;
            int64_t m, c;
            if (kind == 0) { m = rnd() % 5000; c = 1; }
            else if (kind == 1) { m = rnd() % 40; c = 1 + rnd() % 70000; }
            else if (kind == 2) { m = 0; c = rnd() % 9; }
            else { m = rnd() % 600; c = rnd() % 700; }
            s.push_back(m);
            s.push_back(c);
        }
        if (check_plan(s, ws, (int)(rnd() % 3))) {
            printf("failed at random list %d (n=%d ws=%d)\n", it, n, ws);
            return 1;
        }
        plans++;
    }
    printf("ok %d plans\n", plans);
    return 0;
}
