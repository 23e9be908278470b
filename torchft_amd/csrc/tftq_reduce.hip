// k_reduce, tftq_reduce and tftq_check_device: fused_reduce_fp8 on gfx950.
//
// Follows torchft/quantization.py:261-428 (kernels) and :638-686 (launcher); design notes in tftq_device.h.

#include <mutex>

#include "tftq_device.h"

// ---------------------------------------------------------------------------
// reduce
// ---------------------------------------------------------------------------
// The new codes of the register-resident rows leave with streaming stores.  A group of 4
// peers writes a fifth of its traffic, and plain stores left that much dirty in the caches:
// on the fp32 pseudo-gradient of a 1.1 B-parameter model (ws = 4) the kernel took 257 us with
// plain and 215 us with streaming stores, and the dequantize launch behind it 913 against
// 880 us; a group of 8 (a ninth of the traffic) measures the same either way, and so does the
// 4-byte store of the new scale, which stays a plain one.
#define STORE_CODES(val, ptr) STORE_STREAM((val), (ptr))
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

// The same without a branch, for lanes that own a whole short row each whose length is not a
// whole number of 16-byte vectors (loads under a condition end up one per basic block with a
// wait in front of each: a row of 3 dwords cost its lane 3 round trips to memory per peer):
// four dword loads at indices clamped into the row, then dwords past the end are cleared.
// Plain loads: the rows of neighbouring lanes share cache lines, as do the loads of one lane.
DEV u32x4 load_codes_clamped(GLOBAL const u32 *payload, int d0, int ndw, int n)
{
    u32x4 w;
    w.x = payload[min(d0, ndw - 1)];
    w.y = payload[min(d0 + 1, ndw - 1)];
    w.z = payload[min(d0 + 2, ndw - 1)];
    w.w = payload[min(d0 + 3, ndw - 1)];
    const int last = ndw - 1 - d0;  // position of the row's last dword in w
    const u32 mask = (n & 3) ? (1u << (8 * (n & 3))) - 1u : 0xFFFFFFFFu;
    w.x = last < 0 ? 0u : last == 0 ? w.x & mask : w.x;
    w.y = last < 1 ? 0u : last == 1 ? w.y & mask : w.y;
    w.z = last < 2 ? 0u : last == 2 ? w.z & mask : w.z;
    w.w = last < 3 ? 0u : last == 3 ? w.w & mask : w.w;
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

// acc[e] += code[e] / s for the 16 codes of w, s given as (r, r_lo).
// FIRST: acc[e] = code[e] / s, for the first peer of a row.  The reference starts from
// zeros (:405) and 0 + q is q for every q but -0, so the sums can only differ when every
// peer contributes -0: then this sum is -0 where the reference has +0.  requant16 makes
// up for that (a negative zero sum is encoded as +0); the row maximum does not see it.
template <bool FIRST = false>
DEV void accumulate16(float (&acc)[16], const u32x4 w, float r, float r_lo)
{
    const u32 ww[4] = {w.x, w.y, w.z, w.w};

#pragma unroll
    for (int t = 0; t < 4; t++) {
        float f[4];
        unpack_fp8x4(ww[t], f);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float q = div_fast(f[e], r, r_lo);
            acc[4 * t + e] = FIRST ? q : acc[4 * t + e] + q;
        }
    }
}

// (acc * s2) / div, left to right (:364).  Without GDIV, inv_div (1 for SUM) is
// the exact inverse of a power of two and multiplying by it is the same
// correctly rounded result.  GDIV: div is not a power of two.  For div < 1024
// the quotient comes from inv_div = RN(1 / div) in three operations,
//     q0 = y * inv_div,  rem = fma(-q0, div, y),  q = fma(rem, inv_div, q0),
// which equals RN(y / div) for every binary32 y whose quotient is not close to
// the subnormal range (tests/exact_quotient.c checks all 2^23 mantissas of y
// against every odd div below 1024; powers of two in div only move exponents).
// Below 2^-100 the steps may round differently, but every |q| < 2^-10 gives the
// code +-0, with the sign of y restored by the copysign (-0 / div = -0).
// IEEE: the plain divide, for larger group sizes (div_mode 3).
template <bool GDIV, bool IEEE = false>
DEV float scale_div(float a, float s2, const KParams &p)
{
    const float y = __builtin_fmaf(a, s2, 0.0f);  // a * s2, and +0 for a sum of -0 (see accumulate16)
    if (!GDIV) return y * p.inv_div;
    if (IEEE) return y / p.div;
    const float q0 = y * p.inv_div;
    const float rem = __builtin_fmaf(-q0, p.div, y);
    return __builtin_copysignf(__builtin_fmaf(rem, p.inv_div, q0), y);
}

// row maximum / div (:340); for a power-of-two div the multiplication by the
// exact inverse is the same correctly rounded value, subnormal results included
template <bool GDIV>
DEV float amax_div(float amax, const KParams &p)
{
    return GDIV ? amax / p.div : amax * p.inv_div;
}

template <bool GDIV>
DEV u32x4 requant16(const float (&a)[16], float s2, const KParams &p)
{
    float y[16];
    // Power-of-two div: s2 * inv_div is exact unless it is subnormal, and then
    // a * (s2 * inv_div) rounds the same exact product as (a * s2) * inv_div does in two
    // steps; the two can only differ below 2^-126, where every code is zero anyway.
    const float sf = s2 * p.inv_div;
    const bool fold = !GDIV && (sf == 0.0f || __builtin_fabsf(sf) >= 1.17549435e-38f);
    if (__builtin_amdgcn_ballot_w64(!fold) == 0) {  // one code path per wavefront
#pragma unroll
        for (int e = 0; e < 16; e++) y[e] = __builtin_fmaf(a[e], sf, 0.0f);  // a * sf, and +0 for a sum of -0
    } else {
#pragma unroll
        for (int e = 0; e < 16; e++) y[e] = scale_div<GDIV>(a[e], s2, p);
    }
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
template <int TEAM, bool GDIV, bool IEEE = false>
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
                const float y = scale_div<GDIV, IEEE>(a, s2, p);
                orow[4 + c] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, 0.0f, 0, false) & 0xFF);
            }
        }
        if (pass == 0) {
            amax = team_max<TEAM>(amax, lds);
            s2 = calc_scale(amax_div<GDIV>(amax, p));
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
// scales read once.  The second pass reads the peer rows again (from the
// caches if they are still there).
// The passes cover the dwords from d0 on.  The caller deals with the dwords before d0:
// `middle` runs between the first pass and the row maximum and returns their maximum (it
// may read the peers' rows, the own slot included: nothing has been stored yet), `between`
// stores them, when the new scale is known and every lane has finished reading for the
// first pass.  c: division coefficients of peer min(lane, ws - 1), all fast.
// PARK: the sums of the first PARK chunks are parked in LDS (parked: PARK * 16 KB) by the
// first pass and taken from there by the second, which then reads no peer for them.
// A step is a chunk's vectors of up to 8 peers; the loads of the next step are in flight
// while the current one is accumulated (53248 bf16 columns, 8 peers: 62.3 us with steps of 4
// peers one after the other, 56.0 us with steps of 8).
constexpr int R_STEP_PEERS = 8;
template <bool GDIV, int PARK, typename Middle, typename Between>
DEV void reduce_row_two_passes(const Seg &s, const KParams &p, int j, int tid, float *lds, const DivCoef &c,
                               int d0, Middle middle, Between between, float *parked = nullptr)
{
    constexpr int CHUNK = 4 * TFTQ_WG;  // dwords
    const int ndw = (s.row_bytes >> 2) - 1;
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    const int ws = p.ws;  // <= 64 here
    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
    const u32 tailmask = (s.n & 3) ? (1u << (8 * (s.n & 3))) - 1u : 0xFFFFFFFFu;
    const int nchunks = (ndw - d0 + CHUNK - 1) / CHUNK;
    const int nbatches = (ws + R_STEP_PEERS - 1) / R_STEP_PEERS;  // steps per chunk
    float amax = 0.0f, s2 = 0.0f;

    struct Step {
        u32x4 w[R_STEP_PEERS];
    };
    // loads of batch `bi` of chunk `ci`
    auto issue = [&](Step &dst, int ci, int bi) {
        const int doff = min(d0 + ci * CHUNK + 4 * tid, ndw - 4);  // the last vector ends with the row
#pragma unroll
        for (int b = 0; b < R_STEP_PEERS; b++)
            dst.w[b] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(peer_row(p, min(bi * R_STEP_PEERS + b, ws - 1), off) + 1 + doff));
    };
    // what both passes do with the sums of a chunk
    auto finish = [&](const float (&acc)[16], int ci, int pass) {
        const int d = d0 + ci * CHUNK;
        const int doff = min(d + 4 * tid, ndw - 4);
        if (pass == 0) {
#pragma unroll
            for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[e]));
            if (PARK > 0 && ci < PARK) {  // every lane reads back only what it wrote
#pragma unroll
                for (int e = 0; e < 16; e++) parked[(ci * 16 + e) * TFTQ_WG + tid] = acc[e];
            }
        } else {
            // the moved-back last vector overlaps its neighbour, which may sit in another
            // wavefront: nobody stores before everybody has read the own slot's chunk
            __syncthreads();
            if (d + 4 * tid < ndw) {
                const u32x4 o = requant16<GDIV>(acc, s2, p);
                if (doff >= d) {
                    STORE_CODES(o, (GLOBAL u32x4_a4 *)(orow + 1 + doff));
                } else {
                    // The vector reaches back into the dwords before this chunk, whose
                    // codes have already been replaced in the own slot: what was
                    // accumulated for those dwords is meaningless and they are final already.
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (doff + e >= d) orow[1 + doff + e] = o[e];
                }
            }
        }
    };

    auto run_pass = [&](auto pass_c) {
        constexpr int pass = decltype(pass_c)::value;
        float acc[16];
        // the second pass takes the parked chunks from LDS and loads from the first one behind them
        const int first = pass == 0 ? 0 : min(PARK, nchunks);
        if (pass == 1) {
#pragma nounroll
            for (int ci = 0; ci < first; ci++) {
#pragma unroll
                for (int e = 0; e < 16; e++) acc[e] = parked[(ci * 16 + e) * TFTQ_WG + tid];
                finish(acc, ci, 1);
            }
        }
        // steps (chunk, batch) in order; ci, bi: the step to consume, ni, nb: the step to issue
        int ci = first, bi = 0, ni = first, nb = 0;
        auto advance = [&](int &chunk, int &batch) {
            if (++batch == nbatches) {
                batch = 0;
                ++chunk;
            }
        };
        auto consume = [&](const Step &src) {
            const u32 mask = min(d0 + ci * CHUNK + 4 * tid, ndw - 4) == ndw - 4 ? tailmask : 0xFFFFFFFFu;
            if (bi == 0) {
#pragma unroll
                for (int e = 0; e < 16; e++) acc[e] = 0.0f;
            }
#pragma unroll
            for (int b = 0; b < R_STEP_PEERS; b++) {
                const int k = bi * R_STEP_PEERS + b;
                u32x4 w = src.w[b];
                w.w &= mask;
                if (k < ws) accumulate16(acc, w, bcast_lane(c.r, k), bcast_lane(c.r_lo, k));
            }
            if (bi == nbatches - 1) finish(acc, ci, pass);
            advance(ci, bi);
        };
        Step A, B;
        if (ni < nchunks) {
            issue(A, ni, nb);
            advance(ni, nb);
        }
#pragma nounroll
        while (ci < nchunks) {  // A holds the step to consume
            const bool more = ni < nchunks;
            if (more) {
                issue(B, ni, nb);
                advance(ni, nb);
            }
            consume(A);
            if (more) {
                if (ni < nchunks) {
                    issue(A, ni, nb);
                    advance(ni, nb);
                }
                consume(B);
            }
        }
    };
    run_pass(std::integral_constant<int, 0>());
    amax = fmaxf(amax, middle());
    amax = team_max<256>(amax, lds);  // every wavefront has read the old scales by now
    s2 = calc_scale(amax_div<GDIV>(amax, p));
    between(s2);
    run_pass(std::integral_constant<int, 1>());
    if (tid == 0) orow[0] = as_u(s2);  // :375
}

template <bool GDIV>
DEV void reduce_row_long(const Seg &s, const KParams &p, int j, int tid, float *lds)
{
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    const DivCoef c = make_div(guarded_scale(peer_row(p, min(tid & 63, p.ws - 1), off)));
    if (__builtin_amdgcn_ballot_w64(!c.fast) != 0) {  // same in the four wavefronts
        reduce_row_slow<256, GDIV>(s, p, j, tid, lds);
        return;
    }
    reduce_row_two_passes<GDIV, 0>(s, p, j, tid, lds, c, 0, [] { return 0.0f; }, [](float) {});
}

// Wide kernel, rows of more than 8192 payload dwords: the sums of the first 8192
// dwords stay in registers (128 per lane), those of the next 4096 are parked in
// 64 KB of LDS and only the rest of the row makes two passes, so the peers are
// read 1 + rest / length times instead of twice (53248 columns: 1.08 times; with 48 KB of
// LDS 1.15 times and 57.3 instead of 53.4 us).  Two workgroups of 64 KB fit the 160 KB of a
// CU, and the registers admit no more than two.
// The part in registers takes its peers through the rolling window of reduce_rows_roll
// (53248 columns: 65.4 -> 62.3 us against all vectors of a peer loaded, then summed).
constexpr int R_PARKED_CHUNKS = 4;  // chunks of 1024 dwords = 16 KB of sums each
template <bool GDIV>
DEV void reduce_row_hybrid(const Seg &s, const KParams &p, int j, int tid, float *lds, float *parked)
{
    constexpr int UNITS = TFTQ_R_DWORDS_WIDE / (4 * TFTQ_WG);  // 8
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    const int ws = p.ws;  // <= 64 here
    const DivCoef c = make_div(guarded_scale(peer_row(p, min(tid & 63, ws - 1), off)));
    if (__builtin_amdgcn_ballot_w64(!c.fast) != 0) {  // same in the four wavefronts
        reduce_row_slow<256, GDIV>(s, p, j, tid, lds);
        return;
    }
    // The part of the row behind the registers' makes its first pass first (its loads pipelined in
    // registers that the sums of the part in front do not hold yet), then the part in front
    // is summed, then the row maximum is known and both are stored.
    float acc[UNITS][16];  // set by the first peer
    auto front = [&]() {
        // the rolling window of reduce_rows_roll: vector u of the next peer is loaded as soon as
        // vector u of this one has left its registers
        u32x4 w[UNITS];
        {
            GLOBAL const u32 *pv = peer_row(p, 0, off) + 1;
#pragma unroll
            for (int u = 0; u < UNITS; u++) w[u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + 4 * (u * TFTQ_WG + tid)));
        }
        {   // the first peer (a group of one reads it a second time and ignores that)
            const float pr = bcast_lane(c.r, 0), pl = bcast_lane(c.r_lo, 0);
            GLOBAL const u32 *pv = peer_row(p, min(1, ws - 1), off) + 1;
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                u32x4 x = w[u];
                asm volatile("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w));
                w[u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + 4 * (u * TFTQ_WG + tid)));
                accumulate16<true>(acc[u], x, pr, pl);
            }
        }
#pragma nounroll
        for (int k = 1; k + 1 < ws; k++) {
            const float pr = bcast_lane(c.r, k), pl = bcast_lane(c.r_lo, k);
            GLOBAL const u32 *pv = peer_row(p, k + 1, off) + 1;
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                u32x4 x = w[u];
                asm volatile("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w));  // taken out before the registers are loaded again
                w[u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + 4 * (u * TFTQ_WG + tid)));
                accumulate16(acc[u], x, pr, pl);
            }
        }
        if (ws > 1) {
            const float pr = bcast_lane(c.r, ws - 1), pl = bcast_lane(c.r_lo, ws - 1);
#pragma unroll
            for (int u = 0; u < UNITS; u++) accumulate16(acc[u], w[u], pr, pl);
        }
        float amax = 0.0f;
#pragma unroll
        for (int u = 0; u < UNITS; u++)
#pragma unroll
            for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[u][e]));
        return amax;
    };
    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
    reduce_row_two_passes<GDIV, R_PARKED_CHUNKS>(s, p, j, tid, lds, c, TFTQ_R_DWORDS_WIDE, front, [&](float s2) {
#pragma unroll
        for (int u = 0; u < UNITS; u++)
            STORE_CODES(requant16<GDIV>(acc[u], s2, p), (GLOBAL u32x4_a4 *)(orow + 1 + 4 * (u * TFTQ_WG + tid)));
    }, parked);
}

// Register-resident row: the team holds all accumulators of the row, each peer
// row is read once.  UNITS = 16-byte vectors of codes per lane and peer.
// CLAMPED (one lane per row, rows that are not whole 16-byte vectors): loads without branches.
template <int TEAM, int UNITS, bool GDIV, bool CLAMPED = false>
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
                if constexpr (CLAMPED) {
                    // no branch: a peer past the last one re-reads the last and is ignored below
                    GLOBAL const u32 *prow = peer_row(p, min(k0 + b, kend - 1), off);
                    sraw[b] = guarded_scale(prow);
#pragma unroll
                    for (int u = 0; u < UNITS; u++) w[b][u] = load_codes_clamped(prow + 1, u * 4, ndw, n);
                } else if (k0 + b < kend) {
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
    const float s2 = calc_scale(amax_div<GDIV>(amax, p));  // :340

    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
#pragma unroll
    for (int u = 0; u < UNITS; u++)
        store_codes(orow + 1, (u * TEAM + lane) * 4, ndw, requant16<GDIV>(acc[u], s2, p));
    // Every lane read the old scale of the own slot before team_max (wide
    // teams synchronise there; narrow teams are one wavefront in program order).
    if (lane == 0) orow[0] = as_u(s2);  // :375
}

// One row per team, software-pipelined over the peers: the codes of the next
// batch of peers are in flight while the current batch is accumulated.  A
// batch is R_VPB 16-byte vectors per lane: R_VPB / UNITS peers.  Loads carry no
// branch: a lane past the end of the row re-reads the row's last vector, a
// batch past the last peer re-reads the last peer, and both are ignored later.
// Needs ws <= min(TEAM, 64) (lane l of a team, or of each of its wavefronts,
// holds the scale of peer l) and rows of at least one 16-byte vector.  A team
// whose row is past the end (`valid` false) is given the last row and stores
// nothing, so that the wavefront stays converged for the cross-lane operations.
// (Several rows per team with prefetch of the next row were slower for every
// row length: independent workgroups keep more loads in flight.)
constexpr int R_VPB = 4;

template <int TEAM, int UNITS, bool PIPE, bool GDIV, int WS = 0>
DEV void reduce_rows(const Seg &s, const KParams &p, int j, int lane, float *lds, bool valid = true)
{
    constexpr int PB = R_VPB / UNITS >= 1 ? R_VPB / UNITS : 1;  // peers per batch
    const int ndw = (s.row_bytes >> 2) - 1;  // >= 4 here
    // WS: the group size when it is known at compile time (the loops over the peers then
    // unroll into straight-line code); 0: p.ws
    const int ws = WS ? WS : p.ws;
    const int nb = (ws + PB - 1) / PB;  // batches
    const int wlane = TEAM >= 64 ? (int)(threadIdx.x & 63u) : lane;
    const int speer = min(wlane, ws - 1);  // the peer whose scale this lane fetches
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;

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

    // lane l: scale of peer min(l, ws - 1), first in the queue of loads
    const float raw_scale = as_f(peer_row(p, speer, off)[0]);

    struct Batch {
        u32x4 w[PB][UNITS];
    };
    Batch A, B;
    auto issue = [&](Batch &dst, int batch) {
#pragma unroll
        for (int b = 0; b < PB; b++) {
            GLOBAL const u32 *pv = peer_row(p, min(batch * PB + b, ws - 1), off) + 1;
#pragma unroll
            for (int u = 0; u < UNITS; u++)
                dst.w[b][u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + doff[u]));
        }
    };

    issue(A, 0);
    if (PIPE && nb > 1) issue(B, 1);
    // the loads above are issued before anything below: left to itself, the scheduler moves
    // them down between the accumulation steps of the straight-line variants
    __builtin_amdgcn_sched_barrier(0);

    const float sc = raw_scale == 0.0f ? 1.0f : raw_scale;  // padding rows (:419)
    const DivCoef c = make_div(sc);
    if (__builtin_amdgcn_ballot_w64(!c.fast) != 0) {  // same in all wavefronts of the team
        if (valid) reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);  // some peer needs the plain divide
        return;
    }

    float acc[UNITS][16];  // set by the first peer
    auto consume = [&](const Batch &src, int batch, auto first_c) {
        constexpr bool FIRST = decltype(first_c)::value;
#pragma unroll
        for (int b = 0; b < PB; b++) {
            const int k = batch * PB + b;
            if (k < ws) {
                const float pr = team_bcast<TEAM>(c.r, k), pl = team_bcast<TEAM>(c.r_lo, k);
#pragma unroll
                for (int u = 0; u < UNITS; u++) {
                    u32x4 w = src.w[b][u];
                    w.w &= padmask[u];  // here, not at the load: the load must stay in flight
                    if (FIRST && b == 0) accumulate16<true>(acc[u], w, pr, pl);
                    else accumulate16<false>(acc[u], w, pr, pl);
                }
            }
            // peer after peer: work of later peers that is moved up here only holds registers
            if (WS) __builtin_amdgcn_sched_barrier(0);
        }
    };
    const std::true_type first;
    const std::false_type later;

    consume(A, 0, first);
    if (!PIPE) {  // long rows: one batch in flight keeps the register count down
#pragma nounroll
        for (int i = 1; i < nb; i++) {
            issue(A, i);
            consume(A, i, later);
        }
    } else if (WS) {  // straight-line code: batch i in B for odd i, in A for even i
#pragma unroll
        for (int i = 1; i < (WS + PB - 1) / PB; i++) {
            if (i + 1 < (WS + PB - 1) / PB) {
                issue((i & 1) ? A : B, i + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            consume((i & 1) ? B : A, i, later);
        }
    } else {
#pragma nounroll
        for (int i = 1; i < nb; i += 2) {  // B holds batch i
            if (i + 1 < nb) issue(A, i + 1);
            consume(B, i, later);
            if (i + 1 < nb) {
                if (i + 2 < nb) issue(B, i + 2);
                consume(A, i + 1, later);
            }
        }
    }

    float amax = 0.0f;  // duplicates held by lanes past the row's end do not change it
#pragma unroll
    for (int u = 0; u < UNITS; u++)
#pragma unroll
        for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[u][e]));
    amax = team_max<TEAM>(amax, lds);
    const float s2 = calc_scale(amax_div<GDIV>(amax, p));  // :340
    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        const u32x4 o = requant16<GDIV>(acc[u], s2, p);
        if (valid && 4 * (u * TEAM + lane) < ndw) STORE_CODES(o, (GLOBAL u32x4_a4 *)(orow + 1 + doff[u]));
    }
    if (valid && lane == 0) orow[0] = as_u(s2);  // :375; all lanes read the old scale before team_max
}

// Rows of up to 16 * TEAM bytes of codes in teams of 1, 2 or 4 lanes: one vector per lane and
// peer, groups of up to MAXWS (2, 4, 8 or 16) peers, every load of the row in flight at once.  (One
// lane per row reads such a row with two or four loads that lie a row apart from its
// neighbours'; here a load instruction of a wavefront covers 32 or 16 neighbouring rows.)
// Lane l of a team fetches the scales of peers l, l + TEAM, ...: MAXWS / TEAM of them, ahead
// of the codes: a line that a streaming load has brought in is not kept for a later load.
// `valid` as in reduce_rows.
template <int TEAM, int MAXWS, bool GDIV>
DEV void reduce_rows_narrow(const Seg &s, const KParams &p, int j, int lane, float *lds, bool valid)
{
    constexpr int NS = MAXWS > TEAM ? MAXWS / TEAM : 1;  // scales per lane
    const int ndw = (s.row_bytes >> 2) - 1;  // >= 4 here
    const int ws = p.ws;                     // <= MAXWS
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;
    const int doff = min(4 * lane, ndw - 4);  // the last vector ends with the row (see reduce_rows)
    const u32 padmask = (doff == ndw - 4 && (s.n & 3)) ? (1u << (8 * (s.n & 3))) - 1u : 0xFFFFFFFFu;

    float raw[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) raw[i] = as_f(peer_row(p, min(lane + i * TEAM, ws - 1), off)[0]);
    u32x4 w[MAXWS];
#pragma unroll
    for (int k = 0; k < MAXWS; k++)
        w[k] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(peer_row(p, min(k, ws - 1), off) + 1 + doff));
    __builtin_amdgcn_sched_barrier(0);  // all loads are issued before anything below

    DivCoef c[NS];
    bool fast = true;
#pragma unroll
    for (int i = 0; i < NS; i++) {
        c[i] = make_div(raw[i] == 0.0f ? 1.0f : raw[i]);  // padding rows (:419)
        fast = fast && c[i].fast;
    }
    if (__builtin_amdgcn_ballot_w64(!fast) != 0) {
        if (valid) reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);  // some peer needs the plain divide
        return;
    }

    float acc[16];  // set by the first peer
#pragma unroll
    for (int k = 0; k < MAXWS; k++) {
        if (k < ws) {
            const float pr = team_bcast<TEAM>(c[k / TEAM].r, k % TEAM);
            const float pl = team_bcast<TEAM>(c[k / TEAM].r_lo, k % TEAM);
            u32x4 v = w[k];
            v.w &= padmask;
            if (k == 0) accumulate16<true>(acc, v, pr, pl);
            else accumulate16<false>(acc, v, pr, pl);
        }
    }

    float amax = 0.0f;  // duplicates held by lanes past the row's end do not change it
#pragma unroll
    for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[e]));
    amax = team_max<TEAM>(amax, lds);
    const float s2 = calc_scale(amax_div<GDIV>(amax, p));  // :340
    GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
    const u32x4 o = requant16<GDIV>(acc, s2, p);
    if (valid && 4 * lane < ndw) STORE_CODES(o, (GLOBAL u32x4_a4 *)(orow + 1 + doff));
    if (valid && lane == 0) orow[0] = as_u(s2);  // :375; all lanes read the old scale before team_max
}

// One row per team with UNITS >= 2 vectors per lane and peer, as a rolling window over the
// peers: as soon as a lane has taken vector u of peer k out of its registers, the load of
// vector u of peer k + 1 is issued into them, so UNITS loads are in flight all the time at
// the register cost of one peer.  The last peer is peeled off: nothing is loaded behind it.
// Same requirements as reduce_rows.
template <int TEAM, int UNITS, bool GDIV>
DEV void reduce_rows_roll(const Seg &s, const KParams &p, int j, int lane, float *lds, bool valid = true)
{
    const int ndw = (s.row_bytes >> 2) - 1;  // >= 4 here
    const int ws = p.ws;
    const int wlane = TEAM >= 64 ? (int)(threadIdx.x & 63u) : lane;
    const int speer = min(wlane, ws - 1);  // the peer whose scale this lane fetches
    const int64_t off = s.slot_off + (int64_t)j * s.row_bytes;

    u32 boff[UNITS];     // byte offset of vector u of this lane in the payload (see reduce_rows)
    u32 padmask[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        const int d = min(4 * (u * TEAM + lane), ndw - 4);
        boff[u] = 4u * (u32)d;
        padmask[u] = (d == ndw - 4 && (s.n & 3)) ? (1u << (8 * (s.n & 3))) - 1u : 0xFFFFFFFFu;
    }
    const float raw_scale = as_f(peer_row(p, speer, off)[0]);
    u32x4 w[UNITS];
    {
        GLOBAL const uint8_t *pv = (GLOBAL const uint8_t *)(peer_row(p, 0, off) + 1);
#pragma unroll
        for (int u = 0; u < UNITS; u++) w[u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + boff[u]));
    }
    float acc[UNITS][16];  // set by the first peer
    const float sc = raw_scale == 0.0f ? 1.0f : raw_scale;  // padding rows (:419)
    const DivCoef c = make_div(sc);
    const bool row_fast = __builtin_amdgcn_ballot_w64(!c.fast) == 0;  // same in all wavefronts of the team
    if (row_fast) {
        {   // the first peer (a group of one reads it a second time and ignores that)
            const float pr = team_bcast<TEAM>(c.r, 0), pl = team_bcast<TEAM>(c.r_lo, 0);
            GLOBAL const uint8_t *pv = (GLOBAL const uint8_t *)(peer_row(p, min(1, ws - 1), off) + 1);
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                u32x4 x = w[u];
                asm volatile("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w));
                w[u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + boff[u]));
                x.w &= padmask[u];
                accumulate16<true>(acc[u], x, pr, pl);
            }
        }
#pragma nounroll
        for (int k = 1; k + 1 < ws; k++) {
            const float pr = team_bcast<TEAM>(c.r, k), pl = team_bcast<TEAM>(c.r_lo, k);
            GLOBAL const uint8_t *pv = (GLOBAL const uint8_t *)(peer_row(p, k + 1, off) + 1);
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                u32x4 x = w[u];
                asm volatile("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w));  // taken out before the registers are loaded again
                w[u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + boff[u]));
                x.w &= padmask[u];
                accumulate16(acc[u], x, pr, pl);
            }
        }
        if (ws > 1) {
            const float pr = team_bcast<TEAM>(c.r, ws - 1), pl = team_bcast<TEAM>(c.r_lo, ws - 1);
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                u32x4 x = w[u];
                x.w &= padmask[u];
                accumulate16(acc[u], x, pr, pl);
            }
        }
        float amax = 0.0f;  // duplicates held by lanes past the row's end do not change it
#pragma unroll
        for (int u = 0; u < UNITS; u++)
#pragma unroll
            for (int e = 0; e < 16; e++) amax = fmaxf(amax, __builtin_fabsf(acc[u][e]));
        amax = team_max<TEAM>(amax, lds);
        const float s2 = calc_scale(amax_div<GDIV>(amax, p));  // :340
        GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off);
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const u32x4 o = requant16<GDIV>(acc[u], s2, p);
            if (valid && 4 * (u * TEAM + lane) < ndw) STORE_CODES(o, (GLOBAL u32x4_a4 *)((GLOBAL uint8_t *)(orow + 1) + boff[u]));
        }
        if (valid && lane == 0) orow[0] = as_u(s2);  // :375; all lanes read the old scale before team_max
    } else if (valid) {
        reduce_row_slow<TEAM, GDIV>(s, p, j, lane, lds);  // some peer needs the plain divide
    }
}

// Few peers (ws <= 4): ROWS consecutive rows of one team at once, all loads of
// all rows issued together, so that a lane has 8 vectors in flight although a
// row has only ws * UNITS of them.  ws * UNITS * ROWS <= 8.  Rows past the end of
// the tensor are given the last row and store nothing.  lds: 4 * ROWS floats.
template <int TEAM, int UNITS, int ROWS, bool GDIV>
DEV void reduce_rows_at_once(const Seg &s, const KParams &p, int j0, int lane, float *lds)
{
    constexpr int PEERS = 8 / (UNITS * ROWS);  // ws <= PEERS
    const int ndw = (s.row_bytes >> 2) - 1;    // >= 4 here
    const int ws = p.ws;
    const int wlane = (int)(threadIdx.x & 63u);
    const int speer = min(wlane, ws - 1);  // the peer whose scale this lane fetches

    int doff[UNITS];
    u32 padmask[UNITS];  // as in reduce_rows
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        doff[u] = min(4 * (u * TEAM + lane), ndw - 4);
        padmask[u] = (doff[u] == ndw - 4 && (s.n & 3)) ? (1u << (8 * (s.n & 3))) - 1u : 0xFFFFFFFFu;
    }

    int64_t off[ROWS];
    bool valid[ROWS];
    float raw_scale[ROWS];
    u32x4 w[ROWS][PEERS][UNITS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        valid[r] = j0 + r < s.slice_rows;
        off[r] = s.slot_off + (int64_t)min(j0 + r, s.slice_rows - 1) * s.row_bytes;
        raw_scale[r] = as_f(peer_row(p, speer, off[r])[0]);
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int k = 0; k < PEERS; k++) {
            GLOBAL const u32 *pv = peer_row(p, min(k, ws - 1), off[r]) + 1;
#pragma unroll
            for (int u = 0; u < UNITS; u++) w[r][k][u] = LOAD_STREAM((GLOBAL const u32x4_a4 *)(pv + doff[u]));
        }

    float amax[ROWS];
    float acc[ROWS][UNITS][16];
    bool fast[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const float sc = raw_scale[r] == 0.0f ? 1.0f : raw_scale[r];  // padding rows (:419)
        const DivCoef c = make_div(sc);
        fast[r] = __builtin_amdgcn_ballot_w64(!c.fast) == 0;  // same in all wavefronts of the team
#pragma unroll
        for (int u = 0; u < UNITS; u++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[r][u][e] = 0.0f;  // a slow row's sums are not used
        amax[r] = 0.0f;
        if (fast[r]) {
#pragma unroll
            for (int k = 0; k < PEERS; k++) {
                if (k < ws) {
                    const float pr = bcast_lane(c.r, k), pl = bcast_lane(c.r_lo, k);
#pragma unroll
                    for (int u = 0; u < UNITS; u++) {
                        u32x4 v = w[r][k][u];
                        v.w &= padmask[u];
                        if (k == 0) accumulate16<true>(acc[r][u], v, pr, pl);  // the first peer sets the sums
                        else accumulate16(acc[r][u], v, pr, pl);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < UNITS; u++)
#pragma unroll
                for (int e = 0; e < 16; e++) amax[r] = fmaxf(amax[r], __builtin_fabsf(acc[r][u][e]));
        }
    }

    // row maxima over the team: inside the wavefront, then across the four wavefronts
#pragma unroll
    for (int r = 0; r < ROWS; r++) amax[r] = team_max<64>(amax[r], lds);
    if (TEAM == 256) {
        const int wave = threadIdx.x >> 6;
        if (wlane == 0) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) lds[wave * ROWS + r] = amax[r];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < ROWS; r++)
            amax[r] = fmaxf(fmaxf(lds[r], lds[ROWS + r]), fmaxf(lds[2 * ROWS + r], lds[3 * ROWS + r]));
        __syncthreads();
    }

#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        if (fast[r]) {
            const float s2 = calc_scale(amax_div<GDIV>(amax[r], p));  // :340
            GLOBAL u32 *orow = as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off[r]);
#pragma unroll
            for (int u = 0; u < UNITS; u++) {
                const u32x4 o = requant16<GDIV>(acc[r][u], s2, p);
                if (valid[r] && 4 * (u * TEAM + lane) < ndw) STORE_CODES(o, (GLOBAL u32x4_a4 *)(orow + 1 + doff[u]));
            }
            if (valid[r] && lane == 0) orow[0] = as_u(s2);  // :375
        } else if (valid[r]) {
            reduce_row_slow<TEAM, GDIV>(s, p, j0 + r, lane, lds);  // some peer needs the plain divide
        }
    }
}

// Rows of one column: 8 bytes per row and peer, one plain divide per peer
// (coefficients for the fast division would cost two), four rows per lane.
template <bool GDIV, bool IEEE = false>
DEV void reduce_col1(const Seg &s, const KParams &p, int j0, int tid)
{
    // a wavefront none of whose lanes has a row (rows go up with k) leaves at once
    if (__builtin_amdgcn_ballot_w64(j0 + tid < s.slice_rows) == 0) return;
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
            const float s2 = calc_scale(amax_div<GDIV>(fmaxf(0.0f, __builtin_fabsf(acc[k])), p));  // NaN ignored (:331-338)
            u32x2 o;
            o.x = as_u(s2);
            o.y = pack_fp8x4(scale_div<GDIV, IEEE>(acc[k], s2, p), 0.0f, 0.0f, 0.0f) & 0xFFu;
            // streaming: neighbouring lanes write neighbouring rows, whole lines per wavefront
            STORE_STREAM(o, (GLOBAL u32x2_a4 *)as_global<u32>(p.packed + (int64_t)p.rank * p.slot_size + off[k]));
        }
    }
}

// reduce_rows for a team of TEAM lanes with UNITS vectors per lane and peer: groups of 8 and
// of 4 peers run straight-line code (averages over such groups never need GDIV)
#define TFTQ_REDUCE_ROWS(TEAM, UNITS, ...)                                                        \
    do {                                                                                          \
        if (!GDIV && p.ws == 8) reduce_rows<TEAM, UNITS, true, GDIV, GDIV ? 0 : 8>(__VA_ARGS__);  \
        else if (!GDIV && p.ws == 4) reduce_rows<TEAM, UNITS, true, GDIV, GDIV ? 0 : 4>(__VA_ARGS__); \
        else reduce_rows<TEAM, UNITS, true, GDIV>(__VA_ARGS__);                                   \
    } while (0)

// reduce_rows_narrow for a team of TEAM lanes, for the smallest of 2, 4, 8 and 16 peers that
// holds the group (a variant for more peers loads the last peer again in their place)
#define TFTQ_REDUCE_NARROW(TEAM, ...)                                             \
    do {                                                                          \
        if (p.ws <= 2) reduce_rows_narrow<TEAM, 2, GDIV>(__VA_ARGS__);            \
        else if (p.ws <= 4) reduce_rows_narrow<TEAM, 4, GDIV>(__VA_ARGS__);       \
        else if (p.ws <= 8) reduce_rows_narrow<TEAM, 8, GDIV>(__VA_ARGS__);       \
        else reduce_rows_narrow<TEAM, 16, GDIV>(__VA_ARGS__);                     \
    } while (0)

// FLAVOUR: R_ALL, every kind of row; R_WIDE, for lists with rows of more than 16384 columns:
// every kind, twice the registers, half the resident wavefronts; R_LONG, for lists whose rows
// all run in teams of 64 or 256 lanes or have one column (a layer bucket: matrices, norm
// weights, biases): only those kinds.  What
// the compiler makes of one kind's code depends on what else the kernel holds (registers
// kept across the switch, the order of the blocks): with R_LONG the code for the long rows
// of such lists is compiled on its own and does not move when another kind's code changes.
enum { R_ALL = 0, R_WIDE = 1, R_LONG = 2 };
DEV int long_kind(int kind) { return kind == K_GEN64 ? K_GEN64 : kind == K_COL1 ? K_COL1 : K_GEN256; }
template <bool INLINE, bool GDIV, int FLAVOUR>
__global__ __launch_bounds__(TFTQ_WG, FLAVOUR == R_WIDE ? 2 : 4) void k_reduce(const KParams p, const InlineTable inl)
{
    constexpr bool WIDE = FLAVOUR == R_WIDE;
    __shared__ float lds[16];
    __shared__ float parked[WIDE ? R_PARKED_CHUNKS * 16 * TFTQ_WG : 1];  // wide kernel: 64 KB (two workgroups per CU fit)
    Seg s;
    int vb;
    if (!locate<INLINE, ST_R>(p, inl, s, vb)) return;
    int blk = vb - s.wg_begin[ST_R];
    int tid = threadIdx.x;
    if (!INLINE && p.pieces) {
        // vb is a quarter of a workgroup (tftq_reduce_pieces in tftq_internal.h): this wavefront is
        // wavefront blk % 4 of workgroup blk / 4 of its tensor, whatever its neighbours work on
        tid = (blk & 3) * 64 + (tid & 63);
        blk >>= 2;
    }
    const int ndw = (s.row_bytes >> 2) - 1;
    if (GDIV && p.div_mode == 3) {
        // averages over 1024 peers or more, not a power of two: the untuned path with plain divides
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        switch (FLAVOUR == R_LONG ? long_kind(s.kind[ST_R]) : s.kind[ST_R]) {
        case K_GEN256: reduce_row_slow<256, true, true>(s, p, blk, tid, lds); break;
        case K_GEN64:
            if (blk * 4 + wave < s.slice_rows) reduce_row_slow<64, true, true>(s, p, blk * 4 + wave, tid & 63, lds);
            break;
        case K_GEN32:
            if (blk * 8 + (tid >> 5) < s.slice_rows) reduce_row_slow<32, true, true>(s, p, blk * 8 + (tid >> 5), tid & 31, lds);
            break;
        case K_GEN16:
            if (blk * 16 + (tid >> 4) < s.slice_rows) reduce_row_slow<16, true, true>(s, p, blk * 16 + (tid >> 4), tid & 15, lds);
            break;
        case K_GEN8:
            if (blk * 32 + (tid >> 3) < s.slice_rows) reduce_row_slow<8, true, true>(s, p, blk * 32 + (tid >> 3), tid & 7, lds);
            break;
        case K_GEN4:
            if (blk * 64 + (tid >> 2) < s.slice_rows) reduce_row_slow<4, true, true>(s, p, blk * 64 + (tid >> 2), tid & 3, lds);
            break;
        case K_GEN2:
            if (blk * 128 + (tid >> 1) < s.slice_rows) reduce_row_slow<2, true, true>(s, p, blk * 128 + (tid >> 1), tid & 1, lds);
            break;
        case K_GEN1:
            if (blk * 256 + tid < s.slice_rows) reduce_row_slow<1, true, true>(s, p, blk * 256 + tid, 0, lds);
            break;
        case K_COL1: reduce_col1<true, true>(s, p, blk * tftq_col1_rows_per_wg(ST_R), tid); break;
        default: break;
        }
        return;
    }
    // (R_LONG: one of the three kinds that it is launched for, whatever the table says)
    switch (FLAVOUR == R_LONG ? long_kind(s.kind[ST_R]) : s.kind[ST_R]) {
    case K_GEN256: {  // one workgroup per row, or per 2 or 4 rows when the group is small
        const int rows = tftq_reduce_rows_at_once(K_GEN256, ndw, p.ws);
        const int j = blk * rows;
        if (rows == 4) {
            reduce_rows_at_once<256, 1, 4, GDIV>(s, p, j, tid, lds);
        } else if (rows == 2) {
            if (ndw <= 1024) reduce_rows_at_once<256, 1, 2, GDIV>(s, p, j, tid, lds);
            else reduce_rows_at_once<256, 2, 2, GDIV>(s, p, j, tid, lds);
        } else if (WIDE && ndw > TFTQ_R_DWORDS && ndw <= TFTQ_R_DWORDS_WIDE && p.ws <= 64) {
            // vectors per lane and peer that this wavefront needs (see below): 4 to 8
            const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const int nu = min((ndw + 1023) >> 10, (ndw - 256 * wave + 1023) >> 10);
            if (nu <= 4) reduce_rows_roll<256, 4, GDIV>(s, p, j, tid, lds);
            else if (nu == 5) reduce_rows_roll<256, 5, GDIV>(s, p, j, tid, lds);
            else if (nu == 6) reduce_rows_roll<256, 6, GDIV>(s, p, j, tid, lds);
            else if (nu == 7) reduce_rows_roll<256, 7, GDIV>(s, p, j, tid, lds);
            else reduce_rows_roll<256, 8, GDIV>(s, p, j, tid, lds);
        } else if (ndw > TFTQ_R_DWORDS) {
            if (p.ws > 64) reduce_row_slow<256, GDIV>(s, p, j, tid, lds);
            else if (WIDE && ndw > TFTQ_R_DWORDS_WIDE) reduce_row_hybrid<GDIV>(s, p, j, tid, lds, parked);
            else reduce_row_long<GDIV>(s, p, j, tid, lds);
        } else if (p.ws > 64) {
            if (ndw <= 1024) reduce_row<256, 1, GDIV>(s, p, j, tid, lds);
            else reduce_row<256, 4, GDIV>(s, p, j, tid, lds);
        } else {
            // Vectors per lane and peer that this wavefront needs: lane l of the team holds
            // dwords 4 * (256 * u + l) ..., so the upper wavefronts of a row whose length is
            // not a multiple of 1024 dwords need one vector less than the lower ones
            // (10240 columns: 3, 3, 2, 2 instead of 3 each: 55.0 -> 50.4 us on [20480, 10240]).
            // Every variant passes the team's barriers the same number of times.
            const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            // (at least one: a wavefront past the end of a short row still takes part in the barriers)
            const int nu = max(1, min((ndw + 1023) >> 10, (ndw - 256 * wave + 1023) >> 10));
            if (nu == 1) TFTQ_REDUCE_ROWS(256, 1, s, p, j, tid, lds);
            // rows of three or four vectors per lane run the rolling window in all their wavefronts
            // ([20480, 10240]: 53.5 -> 50.4 us against the pipeline in the upper two); rows of two
            // are faster in the pipeline (5120 columns: 50.9 against 62.1 us)
            else if (nu == 2 && ndw > 2048) reduce_rows_roll<256, 2, GDIV>(s, p, j, tid, lds);
            else if (nu == 2) TFTQ_REDUCE_ROWS(256, 2, s, p, j, tid, lds);
            else if (nu == 3) reduce_rows_roll<256, 3, GDIV>(s, p, j, tid, lds);
            else reduce_rows_roll<256, 4, GDIV>(s, p, j, tid, lds);
        }
        break;
    }
    case K_GEN64: {  // one wavefront per row, or per 2 or 4 rows when the group is small
        const int rows = tftq_reduce_rows_at_once(K_GEN64, ndw, p.ws);
        const int j = (blk * 4 + __builtin_amdgcn_readfirstlane(tid >> 6)) * rows;
        if (j >= s.slice_rows) break;  // the whole wavefront leaves
        if (rows == 4) {
            reduce_rows_at_once<64, 1, 4, GDIV>(s, p, j, tid & 63, lds);
        } else if (rows == 2) {
            if (ndw <= 256) reduce_rows_at_once<64, 1, 2, GDIV>(s, p, j, tid & 63, lds);
            else reduce_rows_at_once<64, 2, 2, GDIV>(s, p, j, tid & 63, lds);
        } else if (p.ws > 64) {
            if (ndw <= 256) reduce_row<64, 1, GDIV>(s, p, j, tid & 63, lds);
            else if (ndw <= 512) reduce_row<64, 2, GDIV>(s, p, j, tid & 63, lds);
            else reduce_row_slow<64, GDIV>(s, p, j, tid & 63, lds);
        } else if (ndw <= 256) {
            TFTQ_REDUCE_ROWS(64, 1, s, p, j, tid & 63, lds);
        } else if (ndw <= 512) {
            TFTQ_REDUCE_ROWS(64, 2, s, p, j, tid & 63, lds);
        } else {
            reduce_rows_roll<64, 3, GDIV>(s, p, j, tid & 63, lds);
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
            if (ndw > 4 * TEAM) {  // three vectors per lane (see pick_reduce_kind)
                if (p.ws <= TEAM) reduce_rows_roll<TEAM, 3, GDIV>(s, p, min(j, s.slice_rows - 1), tid % TEAM, lds, j < s.slice_rows);
                else if (j < s.slice_rows) reduce_row_slow<TEAM, GDIV>(s, p, j, tid % TEAM, lds);
            } else if (p.ws <= TEAM) {
                TFTQ_REDUCE_ROWS(TEAM, 1, s, p, min(j, s.slice_rows - 1), tid % TEAM, lds, j < s.slice_rows);
            } else {
                reduce_row<TEAM, 1, GDIV>(s, p, j, tid % TEAM, lds);
            }
        };
        if (s.kind[ST_R] == K_GEN32) small(std::integral_constant<int, 32>());
        else if (s.kind[ST_R] == K_GEN16) small(std::integral_constant<int, 16>());
        else small(std::integral_constant<int, 8>());
        break;
    }
    case K_GEN4: {  // one row per team of 4 lanes, groups of up to 16 peers
        const int j = blk * 64 + (tid >> 2);
        TFTQ_REDUCE_NARROW(4, s, p, min(j, s.slice_rows - 1), tid & 3, lds, j < s.slice_rows);
        break;
    }
    case K_GEN2: {  // one row per pair of lanes, groups of up to 16 peers
        const int j = blk * 128 + (tid >> 1);
        TFTQ_REDUCE_NARROW(2, s, p, min(j, s.slice_rows - 1), tid & 1, lds, j < s.slice_rows);
        break;
    }
    case K_GEN1:  // one lane per row: 1, 2 or 4 vectors of codes per peer
        if (ndw == 4 && p.ws <= 16) {  // one whole vector, all peers in flight at once
            const int j = blk * 256 + tid;
            TFTQ_REDUCE_NARROW(1, s, p, min(j, s.slice_rows - 1), 0, lds, j < s.slice_rows);
        } else if (ndw & 3) {  // not whole 16-byte vectors
            if (ndw <= 4) reduce_row<1, 1, GDIV, true>(s, p, blk * 256 + tid, 0, lds);
            else if (ndw <= 8) reduce_row<1, 2, GDIV, true>(s, p, blk * 256 + tid, 0, lds);
            else reduce_row<1, 4, GDIV, true>(s, p, blk * 256 + tid, 0, lds);
        } else {
            if (ndw <= 4) reduce_row<1, 1, GDIV>(s, p, blk * 256 + tid, 0, lds);
            else if (ndw <= 8) reduce_row<1, 2, GDIV>(s, p, blk * 256 + tid, 0, lds);
            else reduce_row<1, 4, GDIV>(s, p, blk * 256 + tid, 0, lds);
        }
        break;
    case K_COL1: reduce_col1<GDIV>(s, p, blk * tftq_col1_rows_per_wg(ST_R), tid); break;
    default: break;
    }
}

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
// The launch of tftq_reduce with the device already current.
static int reduce_launch(const tftq_plan *plan, const void *table, void *packed, int64_t packed_bytes, int rank,
                         int is_avg, hipStream_t st)
{
    KParams kp;
    InlineTable inl = {};
    bool use_inline;
    int rc = fill_params(plan, ST_R, nullptr, table, nullptr, packed, packed_bytes, st, &kp, &inl, &use_inline);
    if (rc) return rc;
    if (rank < 0 || rank >= plan->ws) return TFTQ_E_ARG;
    kp.rank = rank;
    if (is_avg) {
        const int ws = plan->ws;
        kp.div = (float)ws;
        if ((ws & (ws - 1)) == 0) {
            kp.div_mode = 1;
            kp.inv_div = 1.0f / (float)ws;
        } else if (ws < 1024) {
            kp.div_mode = 2;
            kp.inv_div = 1.0f / (float)ws;
        } else {
            kp.div_mode = 3;
        }
    }
    if (kp.nwg == 0) return 0;
    const unsigned grid = grid_of(kp);
    const bool gdiv = kp.div_mode >= 2;
#define TFTQ_LAUNCH_R(I, G, F) return launch_kernel(k_reduce<I, G, F>, grid, 0, st, kp, inl)
#define TFTQ_LAUNCH_R_FLAVOUR(F)                                                                        \
    do {                                                                                                \
        if (gdiv) { if (use_inline) TFTQ_LAUNCH_R(true, true, F); else TFTQ_LAUNCH_R(false, true, F); } \
        else { if (use_inline) TFTQ_LAUNCH_R(true, false, F); else TFTQ_LAUNCH_R(false, false, F); }    \
    } while (0)
    if (plan->wide[ST_R]) TFTQ_LAUNCH_R_FLAVOUR(R_WIDE);
    else if (plan->reduce_long_rows) TFTQ_LAUNCH_R_FLAVOUR(R_LONG);
    else TFTQ_LAUNCH_R_FLAVOUR(R_ALL);
#undef TFTQ_LAUNCH_R_FLAVOUR
#undef TFTQ_LAUNCH_R
}

extern "C" int tftq_reduce(const tftq_plan *plan, const void *table, void *packed, int64_t packed_bytes, int rank,
                           int is_avg, int device, void *stream)
{
    DeviceScope scope(device);
    if (scope.err != hipSuccess) return (int)scope.err;
    return reduce_launch(plan, table, packed, packed_bytes, rank, is_avg, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------
// tftq_reduce_static: the descriptor table in a fixed array of the code object
// ---------------------------------------------------------------------------
// Every device the library runs on holds its own copy of this array at its own address.
// Host code never uses the array's name as an address: it asks the runtime for the address
// on the current device once (static_table_entry) and uses that pointer from then on.
static __device__ __align__(256) uint8_t static_table[TFTQ_STATIC_TABLE_BYTES];

constexpr int MAX_DEVICES = 64;
// Per device ordinal: the array's address there, and what guards it.  All calls on a device
// share the array, so a call must not rewrite it while the kernel of an earlier call, on
// another stream, may still read it: `done` is recorded behind every reduce kernel, and a
// call on another stream that finds it unfinished returns TFTQ_E_BUSY instead of racing.
// Calls on one stream are ordered by the stream.  Calls that a stream capture records run
// when the graph runs, which this library does not see: they are neither checked nor
// remembered, and serialising them stays with the caller.
struct StaticTable {
    void *ptr = nullptr;        // 0 = not looked up yet
    hipEvent_t done = nullptr;  // created with the look-up
    hipStream_t last = nullptr; // stream of the last call that was not captured
    bool used = false;
    std::mutex in_call;         // one call at a time writes the array and queues its kernel
};
static StaticTable static_tables[MAX_DEVICES];
static std::mutex static_table_mutex;

// The entry of the device that is current on the calling thread, looked up on first use.
static int static_table_entry(StaticTable **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TFTQ_E_ARG;
    StaticTable &t = static_tables[dev];
    std::lock_guard<std::mutex> guard(static_table_mutex);
    if (!t.ptr) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_table));
        if (e != hipSuccess) return (int)e;
        if (!p) return TFTQ_E_ARG;
        hipEvent_t ev = nullptr;
        e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
        if (e != hipSuccess) return (int)e;
        t.done = ev;
        t.ptr = p;
    }
    *out = &t;
    return 0;
}

// Set-up for the current device (called by tftq_check_device).
int tftq_static_table_setup(void)
{
    StaticTable *t = nullptr;
    return static_table_entry(&t);
}

extern "C" int tftq_reduce_static(const tftq_plan *plan, void *packed, int64_t packed_bytes, int rank, int is_avg,
                                  int device, void *stream)
{
    if (!plan) return TFTQ_E_ARG;
    DeviceScope scope(device);
    if (scope.err != hipSuccess) return (int)scope.err;
    hipStream_t st = (hipStream_t)stream;
    if (plan->nseg <= TFTQ_N_INLINE || plan->nwg[ST_R] == 0)  // descriptors in the kernel arguments: no scratch
        return reduce_launch(plan, nullptr, packed, packed_bytes, rank, is_avg, st);
    if (plan->blob.size() > (size_t)TFTQ_STATIC_TABLE_BYTES) return TFTQ_E_TOOBIG;
    if (packed_bytes != plan->output_size) return TFTQ_E_SIZE;  // before anything is queued
    if (rank < 0 || rank >= plan->ws || (!packed && plan->output_size != 0) || ((uintptr_t)packed & 3) != 0)
        return TFTQ_E_ARG;
    StaticTable *t = nullptr;
    int rc = static_table_entry(&t);
    if (rc) return rc;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    hipError_t e = hipStreamIsCapturing(st, &capture);
    if (e != hipSuccess) return (int)e;
    const bool captured = capture != hipStreamCaptureStatusNone;
    std::lock_guard<std::mutex> guard(t->in_call);
    if (!captured && t->used && t->last != st) {
        e = hipEventQuery(t->done);
        if (e == hipErrorNotReady) return TFTQ_E_BUSY;  // an earlier call's kernel, on another stream, may still read the array
        if (e != hipSuccess) return (int)e;
    }
    // the whole image every time: the array keeps whatever the last call, of any plan, left there
    rc = tftq_put_bytes(t->ptr, plan->blob.data(), plan->blob.size(), st);
    if (rc) return rc;
    rc = reduce_launch(plan, t->ptr, packed, packed_bytes, rank, is_avg, st);
    if (!captured) {
        // also after a failed launch: the table kernels above are queued and write the array
        e = hipEventRecord(t->done, st);
        if (e != hipSuccess) return rc ? rc : (int)e;
        t->last = st;
        t->used = true;
    }
    return rc;
}
