/* CPU oracle for the HQMQ KV-cache path, scalar C.  TEST INFRASTRUCTURE ONLY.
 *
 * A second, independent restatement of the reference arithmetic (the first is
 * oracle/torch_oracle.py): every operation is written out with the rounding
 * the reference's torch CPU ops perform, so the result does not depend on the
 * host's BLAS/oneDNN.  Only tests, the smoke check and the benchmark's CPU leg
 * may load this library; the product package never does.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   orc_cell24        src/quantizers/spherical.py:22-43
 *   quat_mul_d        src/quantizers/hqmq.py:33-41
 *   orc_joint_table   src/quantizers/hqmq.py:119-143
 *   orc_quantize      src/quantizers/hqmq.py:145-158,164-169,208-216
 *   orc_med3x         src/quantizers/outlier_aware.py:56-72
 *   orc_outlier_merge src/quantizers/outlier_aware.py:86
 *   orc_dequant       src/quantizers/hqmq_attention.py:39-65
 *   orc_attention     src/quantizers/hqmq_attention.py:68-101 (softmax(QK^T*scale)V in double)
 *   orc_pack_*        no counterpart: the bit-packed cache layout is this build's own
 *
 * Arithmetic model (D = dtype of the tensor being quantized):
 *   a (op) b in D       = RNE_D( fp32(a) (op) fp32(b) )
 *   norm of a 4-chunk   = RNE_D( sqrtf( ((a*a + b*b) + c*c) + d*d ) ), fp32, no FMA
 *   similarity          = RNE_D( fma(u3,j3, fma(u2,j2, fma(u1,j1, u0*j0))) ), fp32
 *   argmax              = first index of the maximum, NaN counts as maximum
 *   round()             = round half to even
 *   quantile(0.5)       = lerp of the two middle order statistics in fp32
 *
 * Pinning: tests/test_oracle_*.py check every function here against the golden
 * fixtures written from the reference and against the torch restatement.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 };

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- fp16 / bf16 <-> fp32, round to nearest even ---- */
static float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        float f = (float)man * (1.0f / 16777216.0f); /* man * 2^-24 */
        return sign ? -f : f;
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112) << 23) | (man << 13));
}
static uint16_t float_to_half(float f) {
    uint32_t x = f2u(f), sign = (x >> 16) & 0x8000u, ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0));
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);        /* rounds to >= 65520 -> inf */
    if (ax < 0x38800000u) {                                          /* subnormal half or zero */
        if (ax < 0x33000000u) return (uint16_t)sign;                 /* < 2^-25 -> 0 (ties handled below) */
        uint32_t e = ax >> 23, m = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126 - e;                                    /* 14..24 */
        uint32_t q = m >> shift, rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (q & 1))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t m = ax + 0xc8000000u;                                   /* rebias exponent by -112 */
    uint32_t q = m >> 13, rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1))) q++;
    return (uint16_t)(sign | q);
}
static float bf16_to_float(uint16_t b) { return u2f((uint32_t)b << 16); }
static uint16_t float_to_bf16(float f) {
    uint32_t x = f2u(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    return (uint16_t)((x + 0x7fffu + lsb) >> 16);
}

static inline float rnd(int dt, float f) {
    if (dt == ORC_F16) return half_to_float(float_to_half(f));
    if (dt == ORC_BF16) return bf16_to_float(float_to_bf16(f));
    return f;
}
static inline int esize(int dt) { return dt == ORC_F32 ? 4 : 2; }
static inline float load_d(int dt, const void *p, size_t i) {
    if (dt == ORC_F16) return half_to_float(((const uint16_t *)p)[i]);
    if (dt == ORC_BF16) return bf16_to_float(((const uint16_t *)p)[i]);
    return ((const float *)p)[i];
}
static inline void store_d(int dt, void *p, size_t i, float f) {
    if (dt == ORC_F16) ((uint16_t *)p)[i] = float_to_half(f);
    else if (dt == ORC_BF16) ((uint16_t *)p)[i] = float_to_bf16(f);
    else ((float *)p)[i] = f;
}

/* exported so tests can check the converters against torch */
void orc_round_array(int dt, const float *in, float *out, long n) { for (long i = 0; i < n; i++) out[i] = rnd(dt, in[i]); }

/* ---- a1: 24-cell ---- */
void orc_cell24(float *out) {
    int r = 0;
    for (int axis = 0; axis < 4; axis++)
        for (int s = 0; s < 2; s++, r++)
            for (int j = 0; j < 4; j++) out[4 * r + j] = (j == axis) ? (s ? -1.0f : 1.0f) : 0.0f;
    for (int m = 0; m < 16; m++, r++)
        for (int j = 0; j < 4; j++) out[4 * r + j] = ((m >> (3 - j)) & 1) ? -0.5f : 0.5f;
}

/* ---- a2: Hamilton product in D, every multiply and every add/sub rounded ---- */
static void quat_mul_d(int dt, const float *a, const float *b, float *o) {
#define M(x, y) rnd(dt, (x) * (y))
#define A(x, y) rnd(dt, (x) + (y))
#define S(x, y) rnd(dt, (x) - (y))
    o[0] = S(S(S(M(a[0], b[0]), M(a[1], b[1])), M(a[2], b[2])), M(a[3], b[3]));
    o[1] = S(A(A(M(a[0], b[1]), M(a[1], b[0])), M(a[2], b[3])), M(a[3], b[2]));
    o[2] = A(A(S(M(a[0], b[2]), M(a[1], b[3])), M(a[2], b[0])), M(a[3], b[1]));
    o[3] = A(S(A(M(a[0], b[3]), M(a[1], b[2])), M(a[2], b[1])), M(a[3], b[0]));
#undef M
#undef A
#undef S
}
void orc_quat_mul(int dt, const float *a, const float *b, float *o) { quat_mul_d(dt, a, b, o); }

static inline float norm4_f32(float a, float b, float c, float d) {
    volatile float s = a * a;      /* volatile: forbid contraction/reassociation */
    volatile float t = b * b; s = s + t;
    t = c * c; s = s + t;
    t = d * d; s = s + t;
    return sqrtf(s);
}

/* ---- a4: joint table, k = p*S + s ---- */
void orc_joint_table(const float *raw, int H, int S, int dt, void *joint) {
    float prim[96];
    orc_cell24(prim);
    for (int h = 0; h < H; h++)
        for (int s = 0; s < S; s++) {
            const float *r = raw + ((size_t)h * S + s) * 4;
            float nrm = norm4_f32(r[0], r[1], r[2], r[3]);
            if (!(nrm >= 1e-8f) && nrm == nrm) nrm = 1e-8f;
            float q[4];
            for (int j = 0; j < 4; j++) q[j] = rnd(dt, r[j] / nrm);
            for (int p = 0; p < 24; p++) {
                float o[4];
                quat_mul_d(dt, prim + 4 * p, q, o);
                for (int j = 0; j < 4; j++) store_d(dt, joint, (((size_t)h * 24 + p) * S + s) * 4 + j, o[j]);
            }
        }
}

static inline float clamp_min_d(int dt, float v, float lo_f32) {
    /* torch clamp(min=c) on a D tensor: NaN propagates, result rounded to D */
    if (v != v) return v;
    float lo = rnd(dt, lo_f32);
    return v < lo ? lo : v;
}

/* ---- a5: quantize.  x (B,H,T,n,4) contiguous in D.  Outputs may be NULL. ---- */
void orc_quantize(const void *x, int dt, long B, int H, long T, int n, const void *joint, int S, int b_r,
                  int32_t *idx_out, int32_t *rq_out, void *rqf_out, void *rmax_out, void *dense_out) {
    const int K = 24 * S;
    const float qmax = (float)((1 << b_r) - 1);
    long rows = B * H * T;
#pragma omp parallel for schedule(static)
    for (long row = 0; row < rows; row++) {
        int h = (int)((row / T) % H);
        float radius[256], rmax = -INFINITY;
        int idx[256];
        int rmax_nan = 0;
        float jt[4];
        for (int c = 0; c < n; c++) {
            size_t base = ((size_t)row * n + c) * 4;
            float v[4], u[4];
            for (int j = 0; j < 4; j++) v[j] = load_d(dt, x, base + j);
            float r = clamp_min_d(dt, rnd(dt, norm4_f32(v[0], v[1], v[2], v[3])), 1e-8f);
            radius[c] = r;
            if (r != r) rmax_nan = 1; else if (r > rmax) rmax = r;
            for (int j = 0; j < 4; j++) u[j] = rnd(dt, v[j] / r);
            int best = 0, best_nan = 0;
            float best_s = 0.f;
            for (int k = 0; k < K; k++) {
                size_t jb = ((size_t)h * K + k) * 4;
                for (int j = 0; j < 4; j++) jt[j] = load_d(dt, joint, jb + j);
                float acc = u[0] * jt[0];
                acc = fmaf(u[1], jt[1], acc);
                acc = fmaf(u[2], jt[2], acc);
                acc = fmaf(u[3], jt[3], acc);
                acc = rnd(dt, acc);
                if (acc != acc) { best = k; best_nan = 1; break; }
                if (k == 0 || acc > best_s) { best = k; best_s = acc; }
            }
            (void)best_nan;
            idx[c] = best;
        }
        float rm = rmax_nan ? NAN : rmax;
        rm = clamp_min_d(dt, rm, 1e-8f);
        float scale = rnd(dt, rm / qmax);
        if (rmax_out) store_d(dt, rmax_out, (size_t)row, rm);
        for (int c = 0; c < n; c++) {
            float q = rnd(dt, radius[c] / scale);
            q = rintf(q);                       /* FE_TONEAREST: half to even */
            if (q == q) { if (q < 0.f) q = 0.f; if (q > qmax) q = qmax; }
            size_t o = (size_t)row * n + c;
            if (idx_out) idx_out[o] = idx[c];
            if (rq_out) rq_out[o] = (q == q) ? (int32_t)q : 0;
            if (rqf_out) store_d(dt, rqf_out, o, q);
            if (dense_out) {
                float rq_scaled = rnd(dt, q * scale);
                size_t jb = ((size_t)h * K + idx[c]) * 4;
                for (int j = 0; j < 4; j++)
                    store_d(dt, dense_out, o * 4 + j, rnd(dt, rq_scaled * load_d(dt, joint, jb + j)));
            }
        }
    }
}

/* ---- a7: Med3x statistics.  mask: 1 byte per chunk. ---- */
static int cmp_float(const void *a, const void *b) {
    float x = *(const float *)a, y = *(const float *)b;
    return (x > y) - (x < y);
}
void orc_med3x(const void *x, int dt, long B, int H, long T, int n, float mult,
               void *norms_out, float *median_out, void *thr_out, uint8_t *mask_out) {
    long per_head = B * T * n;
    float *buf = (float *)malloc(sizeof(float) * (size_t)per_head);
    for (int h = 0; h < H; h++) {
        long m = 0;
        int has_nan = 0;
        for (long b = 0; b < B; b++)
            for (long t = 0; t < T; t++)
                for (int c = 0; c < n; c++) {
                    size_t o = (((size_t)b * H + h) * T + t) * n + c;
                    float v[4];
                    for (int j = 0; j < 4; j++) v[j] = load_d(dt, x, o * 4 + j);
                    float nr = rnd(dt, norm4_f32(v[0], v[1], v[2], v[3]));
                    if (norms_out) store_d(dt, norms_out, o, nr);
                    if (nr != nr) has_nan = 1;
                    buf[m++] = nr;
                }
        float med;
        if (has_nan) med = NAN;
        else {
            qsort(buf, (size_t)per_head, sizeof(float), cmp_float);
            long lo = (per_head - 1) / 2, hi = per_head / 2;   /* floor/ceil of 0.5*(N-1) */
            float a = buf[lo], b2 = buf[hi];
            if (lo == hi) med = a;                             /* weight 0: a + 0*(b-a) */
            else { volatile float d = b2 - a; volatile float e = d * 0.5f; med = b2 - e; }
        }
        median_out[h] = med;
        volatile float t32 = med * mult;
        float thr = rnd(dt, t32);
        if (thr_out) store_d(dt, thr_out, (size_t)h, thr);
        for (long b = 0; b < B; b++)
            for (long t = 0; t < T; t++)
                for (int c = 0; c < n; c++) {
                    size_t o = (((size_t)b * H + h) * T + t) * n + c;
                    float v[4];
                    for (int j = 0; j < 4; j++) v[j] = load_d(dt, x, o * 4 + j);
                    float nr = rnd(dt, norm4_f32(v[0], v[1], v[2], v[3]));
                    mask_out[o] = (nr > thr) ? 1 : 0;
                }
    }
    free(buf);
}

/* torch.where(mask, x, xq) per chunk, raw element copy */
void orc_outlier_merge(const void *x, const void *xq, const uint8_t *mask, int dt, long chunks, void *out) {
    int es = esize(dt) * 4;
    for (long i = 0; i < chunks; i++)
        memcpy((char *)out + (size_t)i * es, (const char *)(mask[i] ? x : xq) + (size_t)i * es, (size_t)es);
}

/* ---- a10: dense decode: joint[h, idx] * ((rq * rs) / qmax), all in D ---- */
void orc_dequant(const int32_t *idx, const int32_t *rq, const void *rs, const void *joint, int dt,
                 long B, int H, long T, int n, int K, int qmax, void *out) {
    long rows = B * H * T;
#pragma omp parallel for schedule(static)
    for (long row = 0; row < rows; row++) {
        int h = (int)((row / T) % H);
        float s = load_d(dt, rs, (size_t)row);
        for (int c = 0; c < n; c++) {
            size_t o = (size_t)row * n + c;
            float r = rnd(dt, rnd(dt, rnd(dt, (float)rq[o]) * s) / (float)qmax);
            size_t jb = ((size_t)h * K + idx[o]) * 4;
            for (int j = 0; j < 4; j++) store_d(dt, out, o * 4 + j, rnd(dt, load_d(dt, joint, jb + j) * r));
        }
    }
}

/* ---- a11: attention over dense K/V (already decoded), double accumulation.
 * Query row i of batch b sees key j iff j < kv_len[b] (or T_kv when kv_len is
 * NULL) and, if causal, j <= i + causal_offset (offset 0 = top-left aligned,
 * the reference's and SDPA's convention). Output fp32. ---- */
void orc_attention(const void *Q, const void *Kd, const void *Vd, int dt, long B, int Hq, int Hkv,
                   long Tq, long Tkv, int d, const int32_t *kv_len, int causal, long causal_offset,
                   double scale, float *out) {
    int g = Hq / Hkv;
    long rows = B * Hq * Tq;
#pragma omp parallel for schedule(static)
    for (long row = 0; row < rows; row++) {
        long b = row / ((long)Hq * Tq);
        int hq = (int)((row / Tq) % Hq);
        long i = row % Tq;
        int hk = hq / g;
        long lim = kv_len ? kv_len[b] : Tkv;
        if (causal && i + causal_offset + 1 < lim) lim = i + causal_offset + 1;
        if (lim > Tkv) lim = Tkv;
        double *sc = (double *)malloc(sizeof(double) * (size_t)(lim > 0 ? lim : 1));
        double mx = -INFINITY;
        for (long j = 0; j < lim; j++) {
            double a = 0;
            size_t kb = (((size_t)b * Hkv + hk) * Tkv + j) * d;
            for (int e = 0; e < d; e++) a += (double)load_d(dt, Q, (size_t)row * d + e) * (double)load_d(dt, Kd, kb + e);
            sc[j] = a * scale;
            if (sc[j] > mx) mx = sc[j];
        }
        double den = 0;
        for (long j = 0; j < lim; j++) { sc[j] = exp(sc[j] - mx); den += sc[j]; }
        for (int e = 0; e < d; e++) {
            double a = 0;
            for (long j = 0; j < lim; j++) a += sc[j] * (double)load_d(dt, Vd, (((size_t)b * Hkv + hk) * Tkv + j) * d + e);
            out[(size_t)row * d + e] = lim > 0 ? (float)(a / den) : 0.f;
        }
        free(sc);
    }
}

/* ---- packed cache rows (this build's layout; see include/hqmq_amd.h).
 * code = idx | rq << idx_bits; low main_bits go to the main plane, the rest to
 * the aux plane; each plane row is a little-endian bit stream over the n
 * chunks of one token. ---- */
static void put_bits(uint8_t *row, long bitpos, uint32_t v, int nbits) {
    for (int i = 0; i < nbits; i++, bitpos++)
        if ((v >> i) & 1u) row[bitpos >> 3] |= (uint8_t)(1u << (bitpos & 7));
}
void orc_pack_rows(const int32_t *idx, const int32_t *rq, long rows, int n, int idx_bits, int main_bits,
                   int aux_bits, uint8_t *main_plane, long main_stride, uint8_t *aux_plane, long aux_stride) {
    for (long r = 0; r < rows; r++) {
        uint8_t *m = main_plane + r * main_stride;
        memset(m, 0, (size_t)main_stride);
        uint8_t *a = aux_bits ? aux_plane + r * aux_stride : NULL;
        if (a) memset(a, 0, (size_t)aux_stride);
        for (int c = 0; c < n; c++) {
            uint32_t code = (uint32_t)idx[r * n + c] | ((uint32_t)rq[r * n + c] << idx_bits);
            put_bits(m, (long)c * main_bits, code & ((1u << main_bits) - 1u), main_bits);
            if (a) put_bits(a, (long)c * aux_bits, code >> main_bits, aux_bits);
        }
    }
}
void orc_pack_flags(const uint8_t *mask, long rows, int n, uint8_t *flags, long stride) {
    for (long r = 0; r < rows; r++) {
        memset(flags + r * stride, 0, (size_t)stride);
        for (int c = 0; c < n; c++)
            if (mask[r * n + c]) flags[r * stride + (c >> 3)] |= (uint8_t)(1u << (c & 7));
    }
}
/* Coordinates of the sideband entries of one (b, h) stream, in the same order: (t & 15) << 8 | c. */
long orc_pack_coords(const uint8_t *mask, long T, int n, uint16_t *coords) {
    long cnt = 0;
    for (long t = 0; t < T; t++)
        for (int c = 0; c < n; c++)
            if (mask[t * n + c]) coords[cnt++] = (uint16_t)(((t & 15) << 8) | c);
    return cnt;
}

/* Sideband for one (b, h) stream: flagged chunks copied in (token, chunk)
 * order; tile_off[i] = number of flagged chunks before token 16*i. Returns the count. */
long orc_pack_sideband(const void *x, const uint8_t *mask, int dt, long T, int n, void *sideband,
                       int32_t *tile_off) {
    long cnt = 0;
    int es = esize(dt) * 4;
    for (long t = 0; t < T; t++) {
        if ((t & 15) == 0) tile_off[t >> 4] = (int32_t)cnt;
        for (int c = 0; c < n; c++)
            if (mask[t * n + c]) {
                memcpy((char *)sideband + (size_t)cnt * es, (const char *)x + (size_t)(t * n + c) * es, (size_t)es);
                cnt++;
            }
    }
    return cnt;
}
