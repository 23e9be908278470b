/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the arithmetic of torchft's FP8 quantized-collective
 * kernels (reference: torchft/quantization.py).  It is the checker that the
 * parity tests, the smoke test and the benchmark's CPU-baseline leg compare
 * the HIP library against; nothing in the shipped package may call it.
 *
 * Arithmetic contract: IEEE-754 binary32 multiply / divide / add with
 * round-to-nearest-even and denormals preserved, fp32 -> OCP e4m3fn with
 * round-to-nearest-even and no saturation (|x| > 464 and NaN/Inf give the NaN
 * code 0x7F | sign), peers summed strictly in the order
 * rank, rank+1, ..., wrapping (quantization.py:405-407).
 *
 * Every function names the reference lines it restates.  How each one is
 * pinned (golden vectors, torch's float8_e4m3fn cast, numpy float16, brute
 * force) is listed in tests/test_oracle.py.  The behaviour of the reference's
 * Triton lowering for NaN/Inf rows and for values above 464 is outside what
 * the reference's sources fix: for those inputs parity is unpinned.
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off -fopenmp)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define TFTQ_F32 0
#define TFTQ_F16 1
#define TFTQ_BF16 2

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ---- element codecs ---------------------------------------------------- */

/* OCP e4m3fn code -> binary32 (exact).  tl.float8e4nv, quantization.py:39. */
float tftq_oracle_e4m3_to_f32(uint8_t c)
{
    uint32_t sign = (uint32_t)(c & 0x80) << 24;
    int e = (c >> 3) & 15, m = c & 7;
    if (e == 15 && m == 7) return u2f(sign | 0x7FC00000u);
    if (e == 0) {
        /* subnormal: m * 2^-9 */
        float v = (float)m * 0.001953125f;
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((uint32_t)(e - 7 + 127) << 23) | ((uint32_t)m << 20));
}

/* binary32 -> e4m3fn, round-to-nearest-even, non-saturating.
 * The cast at quantization.py:156 and :365 (`.to(TL_FP8_TYPE)`). */
uint8_t tftq_oracle_f32_to_e4m3(float x)
{
    uint32_t u = f2u(x);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    u &= 0x7FFFFFFFu;
    if (u > 0x43E80000u) return sign | 0x7F; /* > 464.0, Inf, NaN */
    uint32_t E = u >> 23;
    if (E >= 121) { /* >= 2^-6: normal in e4m3 */
        uint32_t r = u + 0x7FFFFu + ((u >> 20) & 1u);
        r >>= 20;                        /* [exp8 | mant3] */
        r -= (uint32_t)(127 - 7) << 3;   /* rebias */
        return sign | (uint8_t)r;        /* 464 -> rounds to 0x7E (tie, even) */
    }
    /* subnormal target: q = RNE(|x| / 2^-9), 0..8 (8 is the smallest normal) */
    if (E == 0) return sign;
    uint32_t mant = (u & 0x7FFFFFu) | 0x800000u;
    int shift = 141 - (int)E; /* value = mant * 2^(E-150); /2^-9 -> mant * 2^(E-141) */
    if (shift > 24) return sign;
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return sign | (uint8_t)q;
}

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

static inline float f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t e = (h >> 10) & 31, m = h & 0x3FF;
    if (e == 31) return u2f(sign | 0x7F800000u | (m << 13));
    if (e == 0) {
        float v = (float)m * 5.9604644775390625e-08f; /* m * 2^-24 */
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((e - 15 + 127) << 23) | (m << 13));
}

/* binary32 -> bfloat16 RNE: the implicit cast of tl.store, quantization.py:253-257 */
static inline uint16_t f32_to_bf16(float x)
{
    uint32_t u = f2u(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* binary32 -> binary16 RNE: same store cast for fp16 tensors */
static inline uint16_t f32_to_f16(float x)
{
    uint32_t u = f2u(x);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000);
    u &= 0x7FFFFFFFu;
    if (u > 0x7F800000u) return sign | 0x7E00;
    if (u >= 0x477FF000u) return sign | 0x7C00; /* >= 65520 -> Inf (also Inf) */
    uint32_t E = u >> 23;
    if (E >= 113) { /* >= 2^-14: normal */
        uint32_t r = u + 0xFFFu + ((u >> 13) & 1u);
        r >>= 13;
        r -= (uint32_t)(127 - 15) << 10;
        return sign | (uint16_t)r;
    }
    if (E == 0) return sign;
    uint32_t mant = (u & 0x7FFFFFu) | 0x800000u;
    int shift = 126 - (int)E; /* value/2^-24 = mant * 2^(E-126) */
    if (shift > 24) return sign;
    uint32_t q = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return sign | (uint16_t)q;
}

uint16_t tftq_oracle_f32_to_bf16(float x) { return f32_to_bf16(x); }
uint16_t tftq_oracle_f32_to_f16(float x) { return f32_to_f16(x); }
float tftq_oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

static inline int esz_of(int dtype) { return dtype == TFTQ_F32 ? 4 : 2; }

static inline float load_elem(const void *base, int dtype, int64_t idx)
{
    switch (dtype) {
    case TFTQ_F32: return ((const float *)base)[idx];
    case TFTQ_F16: return f16_to_f32(((const uint16_t *)base)[idx]);
    default:       return bf16_to_f32(((const uint16_t *)base)[idx]);
    }
}

static inline void store_elem(void *base, int dtype, int64_t idx, float v)
{
    switch (dtype) {
    case TFTQ_F32: ((float *)base)[idx] = v; break;
    case TFTQ_F16: ((uint16_t *)base)[idx] = f32_to_f16(v); break;
    default:       ((uint16_t *)base)[idx] = f32_to_bf16(v); break;
    }
}

/* ---- scale (quantization.py:44-50) ------------------------------------- */
float tftq_oracle_scale(float row_max)
{
    float s = 448.0f / row_max;
    if (s == u2f(0x7F800000u)) s = 1.0f;
    return s;
}

/* ---- layout (quantization.py:486-503; addressing :108-123) ------------- */
static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* shapes: [T][2] = (m, n).  slot_off: [T] byte offset of tensor i's region
 * inside every slot.  Returns 0, or -1 on bad arguments. */
int tftq_oracle_layout(int T, const int64_t *shapes, int ws,
                       int64_t *slot_off, int64_t *slot_size, int64_t *output_size)
{
    if (T <= 0 || ws <= 0) return -1;
    int64_t per_rank = 0, total = 0;
    for (int i = 0; i < T; i++) {
        int64_t m = shapes[2 * i], n = shapes[2 * i + 1];
        int64_t m_pad = cdiv64(m, ws) * ws;
        int64_t padded = m_pad * (cdiv64(n, 4) + 1) * 4;
        if (slot_off) slot_off[i] = per_rank;
        per_rank += padded / ws;
        total += padded;
    }
    if (slot_size) *slot_size = per_rank;
    if (output_size) *output_size = total;
    return 0;
}

static inline int64_t row_addr(int64_t r, int64_t slice_rows, int64_t slot_size,
                               int64_t slot_off, int64_t row_bytes)
{
    return (r / slice_rows) * slot_size + slot_off + (r % slice_rows) * row_bytes;
}

/* ---- quantize (quantization.py:53-162, 531-588) ------------------------ */
/* ptrs[i] points at element (0,0) of tensor i; strides are element strides
 * [T][2].  `out` (output_size bytes) is zero-filled first, as the reference
 * allocates it with torch.zeros (:567-571). */
int tftq_oracle_quantize(int dtype, int T, const void *const *ptrs,
                         const int64_t *shapes, const int64_t *strides, int ws,
                         uint8_t *out, int nthreads)
{
    int64_t slot_size, output_size;
    int64_t *slot_off = (int64_t *)malloc(sizeof(int64_t) * (size_t)T);
    if (!slot_off) return -2;
    if (tftq_oracle_layout(T, shapes, ws, slot_off, &slot_size, &output_size)) {
        free(slot_off);
        return -1;
    }
    memset(out, 0, (size_t)output_size);
    (void)nthreads;
    for (int i = 0; i < T; i++) {
        const int64_t m = shapes[2 * i], n = shapes[2 * i + 1];
        const int64_t rs = strides[2 * i], cs = strides[2 * i + 1];
        const int64_t slice_rows = cdiv64(m, ws);
        const int64_t row_bytes = (cdiv64(n, 4) + 1) * 4;
        const void *base = ptrs[i];
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nthreads > 0 ? nthreads : 1)
#endif
        for (int64_t r = 0; r < m; r++) {
            float amax = 0.0f;
            for (int64_t c = 0; c < n; c++) {
                /* abs in the input dtype is exact; maximum() ignores NaN (:139) */
                float a = load_elem(base, dtype, r * rs + c * cs);
                a = u2f(f2u(a) & 0x7FFFFFFFu);
                if (a > amax) amax = a;
            }
            float s = tftq_oracle_scale(amax);
            uint8_t *row = out + row_addr(r, slice_rows, slot_size, slot_off[i], row_bytes);
            memcpy(row, &s, 4);
            for (int64_t c = 0; c < n; c++) {
                float x = load_elem(base, dtype, r * rs + c * cs);
                float y = x * s; /* :155, fp32 */
                row[4 + c] = tftq_oracle_f32_to_e4m3(y);
            }
        }
    }
    free(slot_off);
    return 0;
}

/* ---- reduce (quantization.py:261-428, 638-686) ------------------------- */
/* In place on `buf` (ws slots).  Rows 0..slice_rows-1 of every tensor in the
 * own slot are rewritten, padding rows included (:301).  is_avg != 0 selects
 * division_factor = ws (:682), else 1. */
int tftq_oracle_reduce(int T, const int64_t *shapes, int ws, int rank, int is_avg,
                       uint8_t *buf, int nthreads)
{
    int64_t slot_size, output_size;
    int64_t *slot_off = (int64_t *)malloc(sizeof(int64_t) * (size_t)T);
    if (!slot_off) return -2;
    if (rank < 0 || rank >= ws ||
        tftq_oracle_layout(T, shapes, ws, slot_off, &slot_size, &output_size)) {
        free(slot_off);
        return -1;
    }
    const float div = is_avg ? (float)ws : 1.0f;
    (void)nthreads;
    for (int i = 0; i < T; i++) {
        const int64_t m = shapes[2 * i], n = shapes[2 * i + 1];
        const int64_t slice_rows = cdiv64(m, ws);
        const int64_t row_bytes = (cdiv64(n, 4) + 1) * 4;
#ifdef _OPENMP
#pragma omp parallel num_threads(nthreads > 0 ? nthreads : 1)
#endif
        {
            float *acc = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
            for (int64_t j = 0; j < slice_rows; j++) {
                const int64_t off = slot_off[i] + j * row_bytes;
                for (int64_t c = 0; c < n; c++) acc[c] = 0.0f;
                for (int k = 0; k < ws; k++) {
                    const int p = (rank + k) % ws; /* :407 */
                    const uint8_t *prow = buf + (int64_t)p * slot_size + off;
                    float s;
                    memcpy(&s, prow, 4);
                    if (s == 0.0f) s = 1.0f; /* :419 */
                    for (int64_t c = 0; c < n; c++)
                        acc[c] = acc[c] + tftq_oracle_e4m3_to_f32(prow[4 + c]) / s; /* :426 */
                }
                float amax = 0.0f;
                for (int64_t c = 0; c < n; c++) {
                    float a = u2f(f2u(acc[c]) & 0x7FFFFFFFu);
                    if (a > amax) amax = a; /* :334-335 */
                }
                const float s2 = tftq_oracle_scale(amax / div); /* :340 */
                uint8_t *orow = buf + (int64_t)rank * slot_size + off;
                for (int64_t c = 0; c < n; c++) {
                    float y = (acc[c] * s2) / div; /* :364 */
                    orow[4 + c] = tftq_oracle_f32_to_e4m3(y);
                }
                memcpy(orow, &s2, 4); /* :375 */
            }
            free(acc);
        }
    }
    free(slot_off);
    return 0;
}

/* ---- dequantize (quantization.py:165-258, 591-635) --------------------- */
int tftq_oracle_dequantize(int dtype, int T, void *const *ptrs,
                           const int64_t *shapes, const int64_t *strides, int ws,
                           const uint8_t *buf, int nthreads)
{
    int64_t slot_size, output_size;
    int64_t *slot_off = (int64_t *)malloc(sizeof(int64_t) * (size_t)T);
    if (!slot_off) return -2;
    if (tftq_oracle_layout(T, shapes, ws, slot_off, &slot_size, &output_size)) {
        free(slot_off);
        return -1;
    }
    (void)nthreads;
    for (int i = 0; i < T; i++) {
        const int64_t m = shapes[2 * i], n = shapes[2 * i + 1];
        const int64_t rs = strides[2 * i], cs = strides[2 * i + 1];
        const int64_t slice_rows = cdiv64(m, ws);
        const int64_t row_bytes = (cdiv64(n, 4) + 1) * 4;
        void *base = ptrs[i];
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nthreads > 0 ? nthreads : 1)
#endif
        for (int64_t r = 0; r < m; r++) {
            const uint8_t *row = buf + row_addr(r, slice_rows, slot_size, slot_off[i], row_bytes);
            float s;
            memcpy(&s, row, 4); /* :239, no zero guard */
            for (int64_t c = 0; c < n; c++) {
                /* fp8 -> input dtype is exact; the divide is fp32 (:250-252) */
                float v = tftq_oracle_e4m3_to_f32(row[4 + c]) / s;
                store_elem(base, dtype, r * rs + c * cs, v);
            }
        }
    }
    free(slot_off);
    return 0;
}

int tftq_oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

int tftq_oracle_esz(int dtype) { return esz_of(dtype); }
