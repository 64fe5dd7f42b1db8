// HQMQ quantize (+ Med3x mask, + bit-packing) for one K or V tensor.
//
// Follows HQMQQuantizer._qdq, unit-magnitude / linear-radius branch
// (src/quantizers/hqmq.py:145-158,164-169,208-216 of the reference) and the
// mask/merge of OutlierAwareHQMQQuantizer._qdq (src/quantizers/outlier_aware.py:72,86).
//
// One lane per 4-element chunk.  The codeword the reference picks is
//     first k = p*S+s maximising  RNE_D( fma-chain_fp32( u . J[k] ) ),
// u = RNE_D(x / r).  Instead of scoring all 24*S rows, each lane rotates its
// chunk by conj(q_s) (q_s broadcast from LDS): <u, q_p*q_s> = <u*conj(q_s), q_p>,
// and the best Hurwitz unit for a rotated chunk v is closed form
// (max_i |v_i| for the 8 axis units, sum_i |v_i| / 2 for the 16 half units).
// That gives the exact-arithmetic score of the best p for every s in ~25
// operations.  Rounding decides the reference's choice among near-ties, so the
// closed form is only a filter: every (p, s) whose exact score is within a
// proven margin of the best is re-scored with the reference's rounding, and
// the smallest index among the maxima wins.  The margin covers the rounding of
// the joint table (slack[h] from hqmq_build_joint), the final RNE_D of the
// score and the float error of the filter itself.  Lanes whose candidate lists
// overflow, or whose direction is not finite, score all 24*S rows instead.
//
// Compiled with -ffp-contract=off; fused multiply-adds are written explicitly.
#include "common.h"
#include <type_traits>

namespace hqmq {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kQThreads = 256;
constexpr int kSCap = 32;  // candidate secondaries kept per lane
constexpr int kKCap = 24;  // candidate codewords kept per lane

// Maximum over groups of `n` neighbouring lanes (n a power of two up to 64), every lane of a group receiving it:
// lane permutations inside the vector unit (quad, half-row and row mirrors, then the 16- and 32-lane row swaps).
// The operands are ordinary numbers or -inf (no NaN), as unsigned bit patterns of non-negative floats order like the
// values, the same routine serves both.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, false);
}
template <class T, class MAX>
__device__ __forceinline__ T group_max(T x, int n, MAX mx) {
    auto step = [&](uint32_t other) { x = mx(x, __builtin_bit_cast(T, other)); };
    if (n >= 2) step(dpp_u32<0xB1>(__builtin_bit_cast(uint32_t, x)));       // quad_perm [1,0,3,2]
    if (n >= 4) step(dpp_u32<0x4E>(__builtin_bit_cast(uint32_t, x)));       // quad_perm [2,3,0,1]
    if (n >= 8) step(dpp_u32<0x141>(__builtin_bit_cast(uint32_t, x)));      // row_half_mirror
    if (n >= 16) step(dpp_u32<0x140>(__builtin_bit_cast(uint32_t, x)));     // row_mirror
    if (n >= 32) {
        const uint32_t b = __builtin_bit_cast(uint32_t, x);
        const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
        x = mx(__builtin_bit_cast(T, (uint32_t)r[0]), __builtin_bit_cast(T, (uint32_t)r[1]));
    }
    if (n >= 64) {
        const uint32_t b = __builtin_bit_cast(uint32_t, x);
        const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
        x = mx(__builtin_bit_cast(T, (uint32_t)r[0]), __builtin_bit_cast(T, (uint32_t)r[1]));
    }
    return x;
}

struct QParams {
    const void *x;
    int64_t xsb, xsh, xst;
    int B, H, T, n;
    const void *joint;
    const float *slack;
    int S, qmax;
    int32_t *idx_out, *rq_out;
    void *rmax_out, *dense_out;
    const void *thr;
    uint8_t *mask_out;
    uint8_t *main_plane, *aux_plane, *flag_plane;
    void *scale_plane;
    int64_t t_cap;
    int t_off;
    const int32_t *pos;
    int idx_bits, main_bits, aux_bits;
    int tokens_per_block;
    int32_t *stats;
    uint32_t *scale_max;
    // sideband compaction in the same launch (compact != 0): see the end of quantize_body
    int compact;
    void *sideband;
    int64_t sb_cap;
    int32_t *sb_tile_off, *sb_count, *overflow;
    uint16_t *sb_coord;
};

__device__ __forceinline__ void rotate_conj(const float u[4], float qw, float qx, float qy, float qz, float v[4]) {
    // v = u * conj(q)
    v[0] = fmaf(u[3], qz, fmaf(u[2], qy, fmaf(u[1], qx, u[0] * qw)));
    v[1] = fmaf(u[3], qy, fmaf(-u[2], qz, fmaf(u[1], qw, -u[0] * qx)));
    v[2] = fmaf(-u[3], qx, fmaf(u[2], qw, fmaf(u[1], qz, -u[0] * qy)));
    v[3] = fmaf(u[3], qw, fmaf(u[2], qx, fmaf(-u[1], qy, -u[0] * qz)));
}

// twice the exact score of the best Hurwitz unit for rotated chunk v
__device__ __forceinline__ float best2_of(const float v[4]) {
    float a0 = fabsf(v[0]), a1 = fabsf(v[1]), a2 = fabsf(v[2]), a3 = fabsf(v[3]);
    float sum = (a0 + a1) + (a2 + a3);
    float mx = fmaxf(fmaxf(a0, a1), fmaxf(a2, a3));
    return fmaxf(mx + mx, sum);
}

// best2_of on the four results of the rotating MFMA, same values: |.| rides on the operands of v_max / v_max3
// (the compiler's own code quiets every operand with an extra v_max first).  `sum` is also an input of the asm so
// that it is placed behind the compiler's own first reads of the MFMA result.
__device__ __forceinline__ float best2_mfma(float v0, float v1, float v2, float v3) {
    const float sum = (fabsf(v0) + fabsf(v1)) + (fabsf(v2) + fabsf(v3));
    float m23, mx;
    asm("v_max_f32_e64 %0, |%1|, |%2|" : "=v"(m23) : "v"(v2), "v"(v3), "v"(sum));
    asm("v_max3_f32 %0, |%1|, |%2|, %3" : "=v"(mx) : "v"(v0), "v"(v1), "v"(m23));
    return fmaxf(mx + mx, sum);
}

// What the doubled filter score of a secondary must reach for one of its codewords to be able to win, given the
// largest doubled filter score m2 seen so far.  The reference rounds every score once to D.  The unrounded
// reference score of the best codeword is at least x = m2 / 2 less the errors of the filter and of the table, so
// the winning rounded score is at least R = RNE_D(x), and only unrounded scores from the midpoint below R upwards
// round that high.  Taking the table and filter errors off once more turns that midpoint into a bound on the
// filter score.  On average this is half a unit in the last place of D tighter than the worst-case margin, which
// it never undercuts (the larger of the two bounds is returned; both hold).
template <class D>
__device__ __forceinline__ float candidate_threshold(float m2, float table_err, float filter_err, float margin2) {
    const float worst = m2 - margin2;
    if (D::code == HQMQ_F32) return worst;
    const float x = 0.5f * (m2 - 0.5f * filter_err) - table_err;
    const float R = D::rnd(x);
    // R is a normal number of D here, so the number of D below it is one step of D's last mantissa bit down
    const float below = __uint_as_float(__float_as_uint(R) - (D::code == HQMQ_F16 ? 1u << 13 : 1u << 16));
    const float mid = 0.5f * (R + below);
    const float thr = 2.f * (mid - table_err) - 0.5f * filter_err;
    return R > 1.0e-4f ? fmaxf(thr, worst) : worst;
}

// twice the exact score of Hurwitz unit p for rotated chunk v
__device__ __forceinline__ float exact2_of(const float v[4], int p) {
    if (p < 8) {
        float t = v[p >> 1];
        t = t + t;
        return (p & 1) ? -t : t;
    }
    int m = p - 8;
    float t0 = (m & 8) ? -v[0] : v[0], t1 = (m & 4) ? -v[1] : v[1];
    float t2 = (m & 2) ? -v[2] : v[2], t3 = (m & 1) ? -v[3] : v[3];
    return (t0 + t1) + (t2 + t3);
}

template <class D>
__device__ __forceinline__ float ref_score(const float u[4], const typename D::storage *row) {
    float j0 = D::load(row), j1 = D::load(row + 1), j2 = D::load(row + 2), j3 = D::load(row + 3);
    float acc = u[0] * j0;
    acc = fmaf(u[1], j1, acc);
    acc = fmaf(u[2], j2, acc);
    acc = fmaf(u[3], j3, acc);
    return D::rnd(acc);
}

// argmax over all K rows with torch's rule: first maximum, NaN counts as maximum.
template <class D>
__device__ int brute_argmax(const float u[4], const typename D::storage *jh, int K) {
    int best = 0;
    float bs = 0.f;
    for (int k = 0; k < K; k++) {
        float s = ref_score<D>(u, jh + (size_t)k * 4);
        if (is_nan(s)) return k;
        if (k == 0 || s > bs) { bs = s; best = k; }
    }
    return best;
}

// Little-endian bit stream of `w`-bit fields (field i = vals[base + i] >> shift, masked)
// -> output byte `byte` of the row.
template <int W>
__device__ __forceinline__ uint8_t gather_byte_w(const uint32_t *vals, int count, int w, int shift, int byte) {
    const int ww = W ? W : w;       // W != 0: the width is a constant and the divisions below fold into shifts
    uint32_t out = 0;
    uint32_t fmask = (ww >= 32) ? 0xffffffffu : ((1u << ww) - 1u);
#pragma unroll
    for (int bit = 0; bit < 8; bit++) {
        int pos = byte * 8 + bit;
        int i = pos / ww, o = pos - i * ww;
        if (i < count) out |= ((((vals[i] >> shift) & fmask) >> o) & 1u) << bit;
    }
    return (uint8_t)out;
}
__device__ __forceinline__ uint8_t gather_byte(const uint32_t *vals, int count, int w, int shift, int byte) {
    switch (w) {        // the widths the layout rule produces (main 8 / 12, aux 1..3, flags 1)
        case 1: return gather_byte_w<1>(vals, count, w, shift, byte);
        case 2: return gather_byte_w<2>(vals, count, w, shift, byte);
        case 3: return gather_byte_w<3>(vals, count, w, shift, byte);
        case 8: return gather_byte_w<8>(vals, count, w, shift, byte);
        case 12: return gather_byte_w<12>(vals, count, w, shift, byte);
        default: return gather_byte_w<0>(vals, count, w, shift, byte);
    }
}

// SPLIT (single-token appends, 16-bit dtypes, n a power of two): the block's 256 / n token slots all hold the one new
// token of (b, h) and share its secondaries between them: slot w scores s = w, w + slots, ...  A decode-step append is
// one wavefront's serial instruction stream otherwise; this divides the search part of it by the number of slots.
// The slots' candidates are merged exactly: the filter threshold comes from the maximum over all slots, the winner
// is the highest exact score with the lowest index, as in the unsplit search.
template <class D, int ALGO, bool SPLIT = false>
__device__ __forceinline__ void quantize_body(const QParams &a) {
    using ST = typename D::storage;
    static_assert(!SPLIT || (ALGO == 0 && D::code != HQMQ_F32), "the split search is the MFMA search");
    extern __shared__ float sec[];  // [S][4] secondaries, then [S][4] fp16 columns of their rotation matrices
    uint2 *rot = reinterpret_cast<uint2 *>(sec + 4 * a.S);
    __shared__ float radius_sh[kQThreads];
    __shared__ uint32_t code_sh[kQThreads];
    __shared__ uint32_t mask_sh[kQThreads];
    __shared__ uint16_t slist[kSCap][kQThreads];
    __shared__ uint16_t klist[kKCap][kQThreads];

    const int tid = threadIdx.x;
    const int bh = blockIdx.y, b = bh / a.H, h = bh - b * a.H;
    const int n = a.n, S = a.S, K = 24 * S;
    const int tok_local = tid / n, c = tid - tok_local * n;       // SPLIT: tok_local is the slot
    const int t = SPLIT ? (int)blockIdx.x : blockIdx.x * a.tokens_per_block + tok_local;
    const bool active = tok_local < a.tokens_per_block && t < a.T;
    const bool writer = !SPLIT || tok_local == 0;                 // one slot stores the results
    const int slots = SPLIT ? kQThreads / n : 1, s_first = SPLIT ? tok_local : 0;
    const ST *jh = (const ST *)a.joint + (size_t)h * K * 4;

    for (int i = tid; i < S * 4; i += kQThreads) sec[i] = D::load(jh + i);  // rows k = s are q_s itself
    if (ALGO == 0 && D::code != HQMQ_F32) {
        // column i of M(q) with u * conj(q) = u M: (w,x,y,z), (-x,w,-z,y), (-y,z,w,-x), (-z,-y,x,w)
        for (int i = tid; i < S * 4; i += kQThreads) {
            const ST *q = jh + (i >> 2) * 4;
            const float w = D::load(q), x = D::load(q + 1), y = D::load(q + 2), z = D::load(q + 3);
            half4 c;
            switch (i & 3) {
                case 0: c = half4{(_Float16)w, (_Float16)x, (_Float16)y, (_Float16)z}; break;
                case 1: c = half4{(_Float16)-x, (_Float16)w, (_Float16)-z, (_Float16)y}; break;
                case 2: c = half4{(_Float16)-y, (_Float16)z, (_Float16)w, (_Float16)-x}; break;
                default: c = half4{(_Float16)-z, (_Float16)-y, (_Float16)x, (_Float16)w}; break;
            }
            rot[i] = __builtin_bit_cast(uint2, c);
        }
    }

    float xv[4] = {0.f, 0.f, 0.f, 0.f};
    if (active) {
        const ST *xp = (const ST *)a.x + b * a.xsb + h * a.xsh + (int64_t)t * a.xst + c * 4;
        for (int j = 0; j < 4; j++) xv[j] = D::load(xp + j);
    }
    const float nrm = D::rnd(norm4(xv[0], xv[1], xv[2], xv[3]));
    const float r = clamp_min_d<D>(nrm, 1e-8f);
    float u[4];
    for (int j = 0; j < 4; j++) u[j] = D::rnd(xv[j] / r);
    radius_sh[tid] = r;
    __syncthreads();

    // ---- codeword search ----
    int idx = 0;
    const bool finite = fabsf(u[0]) < INFINITY && fabsf(u[1]) < INFINITY && fabsf(u[2]) < INFINITY && fabsf(u[3]) < INFINITY;
    const bool zero = u[0] == 0.f && u[1] == 0.f && u[2] == 0.f && u[3] == 0.f;
    if (ALGO == 1) {
        if (active) idx = brute_argmax<D>(u, jh, K);
    } else {
        bool brute = active && !finite;            // NaN/inf directions: exact emulation only
        const bool search = active && finite && !zero;  // all-zero direction: every score is 0 -> index 0
        float us[4];
        for (int j = 0; j < 4; j++) us[j] = search ? u[j] : (j == 0 ? 1.f : 0.f);
        const float ulen = sqrtf(fmaf(us[3], us[3], fmaf(us[2], us[2], fmaf(us[1], us[1], us[0] * us[0])))) * 1.000001f;
        const float table_err = ulen * (a.slack[h] + 9.5367e-7f);      // unrounded reference score vs exact score
        const float filter_err = ulen * 7.6294e-6f + 1.0e-6f;           // doubled filter score vs twice the exact score
        const float E = table_err + ulen * 1.01f * D::eps();
        const float margin2 = 4.f * E + filter_err;
        float m2 = -INFINITY;
        int cnt = 0;
        if (D::code != HQMQ_F32) {
            // 16-bit dtypes: u and q_s are exact in fp16, so one v_mfma_f32_4x4x4_16B_f16 rotates the 64 chunks
            // of the wavefront by q_s: block = 4 consecutive lanes, A = columns of the rotation matrix (the same
            // for every block, lane i holds column i), B = the lane's own direction, D = its rotated chunk.
            const half4 ub = half4{(_Float16)us[0], (_Float16)us[1], (_Float16)us[2], (_Float16)us[3]};
            const uint2 *acol = rot + (tid & 3);
            // The scan runs in blocks of 32 secondaries whose scores stay in registers.  Only the running maximum is
            // kept inside a block; at its end the secondaries that reach the candidate threshold of the maximum so far
            // become a bit mask (a compare and an add-with-carry each) and go into the list of the re-score below.  A
            // threshold that has moved above the maximum before the block leaves everything listed before below the
            // final threshold: the list starts over.
            const int iters = (S + slots - 1) / slots;          // of the slot with the most secondaries (wave-uniform)
            uint2 a_next = acol[4 * min(s_first, S - 1)];
            float thr = -INFINITY;
            auto scan_block = [&](int i0, auto tail) -> uint32_t {
                float b2v[32];
#pragma unroll
                for (int i = 0; i < 32; i++) {
                    const int sn = s_first + (i0 + i + 1) * slots;
                    const half4 am = __builtin_bit_cast(half4, a_next);
                    // the next column is on its way during this one; inside a whole block it exists, so its address is
                    // the block's base plus a constant
                    a_next = (decltype(tail)::value || i == 31) ? acol[4 * min(sn, S - 1)] : acol[4 * sn];
                    const float4v vv = __builtin_amdgcn_mfma_f32_4x4x4f16(am, ub, float4v{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    float b2 = best2_mfma(vv[0], vv[1], vv[2], vv[3]);
                    if (decltype(tail)::value && sn - slots >= S) b2 = -INFINITY;      // behind the slot's last secondary
                    b2v[i] = b2;
                    // the running maximum takes two scores at a time (all ordinary numbers or -inf here)
                    if (i & 1) asm("v_max3_f32 %0, %1, %2, %3" : "=v"(m2) : "v"(m2), "v"(b2v[i - 1]), "v"(b2));
                }
                thr = candidate_threshold<D>(m2, table_err, filter_err, margin2);
                uint32_t word = 0u;
#pragma unroll
                for (int i = 31; i >= 0; i--)       // word = 2 word + (score >= thr): iteration i ends up in bit i
                    asm("v_cmp_ge_f32_e32 vcc, %1, %2\n\tv_addc_co_u32_e32 %0, vcc, %0, %0, vcc" : "+v"(word) : "v"(b2v[i]), "v"(thr) : "vcc");
                if (decltype(tail)::value) {        // a slot whose secondaries end inside the block: only those count
                    const int left = S - s_first - i0 * slots;
                    const int valid = left <= 0 ? 0 : min((left + slots - 1) / slots, 32);
                    word &= valid >= 32 ? ~0u : (1u << valid) - 1u;
                }
                return word;
            };
            for (int i0 = 0; i0 < iters; i0 += 32) {
                const float m_before = m2;
                const bool whole = (slots - 1) + (i0 + 31) * slots < S;     // every slot has all 32 secondaries of this block
                uint32_t bits = whole ? scan_block(i0, std::false_type{}) : scan_block(i0, std::true_type{});
                if (m_before < thr) cnt = 0;
                while (bits) {
                    const int i = __builtin_ctz(bits);
                    bits &= bits - 1u;
                    if (cnt < kSCap) slist[cnt][tid] = (uint16_t)(s_first + (i0 + i) * slots);
                    cnt++;
                }
            }
        } else {
            for (int s = 0; s < S; s++) {
                const float4 q = *reinterpret_cast<const float4 *>(sec + 4 * s);
                float v[4];
                rotate_conj(us, q.x, q.y, q.z, q.w, v);
                const float b2 = best2_of(v);
                if (b2 + margin2 >= m2) {
                    if (b2 - margin2 > m2) cnt = 0;
                    if (cnt < kSCap) slist[cnt][tid] = (uint16_t)s;
                    cnt++;
                }
                m2 = fmaxf(m2, b2);
            }
        }
        if (SPLIT) {        // the maximum over all slots of this chunk (every slot holds the same direction)
            float *m2_sh = reinterpret_cast<float *>(code_sh);
            m2_sh[tid] = m2;
            __syncthreads();
            for (int w = 0; w < slots; w++) m2 = fmaxf(m2, m2_sh[w * n + c]);
            __syncthreads();
        }
        float bs = -INFINITY;
        int bk = 0x7fffffff;
        if (search) {
            if (cnt > kSCap) brute = true;
            const float thr2 = candidate_threshold<D>(m2, table_err, filter_err, margin2);
            int kcnt = 0;
            if (!brute) {
                for (int i = 0; i < cnt; i++) {
                    const int s = slist[i][tid];
                    const float4 q = *reinterpret_cast<const float4 *>(sec + 4 * s);
                    float v[4];
                    rotate_conj(us, q.x, q.y, q.z, q.w, v);
                    const float a0 = fabsf(v[0]), a1 = fabsf(v[1]), a2 = fabsf(v[2]), a3 = fabsf(v[3]);
                    const float sum = (a0 + a1) + (a2 + a3);
                    const float mx = fmaxf(fmaxf(a0, a1), fmaxf(a2, a3));
                    if (fmaxf(mx + mx, sum) < thr2) continue;  // entered while the running maximum was lower
                    // Usually exactly one Hurwitz unit of this secondary is inside the margin: the largest axis
                    // or the all-signs-matched half unit. Count the others; only then enumerate all 24.
                    const int n_axis = (a0 + a0 >= thr2) + (a1 + a1 >= thr2) + (a2 + a2 >= thr2) + (a3 + a3 >= thr2);
                    const int n_flip = (sum - (a0 + a0) >= thr2) + (sum - (a1 + a1) >= thr2) + (sum - (a2 + a2) >= thr2) +
                                       (sum - (a3 + a3) >= thr2);
                    const int n_half = (sum >= thr2) + n_flip;
                    if (n_axis + n_half == 1) {
                        int pp;
                        if (n_axis) {
                            const int im = (a0 == mx) ? 0 : (a1 == mx) ? 1 : (a2 == mx) ? 2 : 3;
                            const float vm = (a0 == mx) ? v[0] : (a1 == mx) ? v[1] : (a2 == mx) ? v[2] : v[3];
                            pp = 2 * im + (vm < 0.f ? 1 : 0);
                        } else {
                            pp = 8 + ((v[0] < 0.f ? 8 : 0) | (v[1] < 0.f ? 4 : 0) | (v[2] < 0.f ? 2 : 0) | (v[3] < 0.f ? 1 : 0));
                        }
                        if (kcnt < kKCap) klist[kcnt][tid] = (uint16_t)(pp * S + s);
                        kcnt++;
                    } else {
#pragma unroll
                        for (int p = 0; p < 24; p++) {
                            if (exact2_of(v, p) >= thr2) {
                                if (kcnt < kKCap) klist[kcnt][tid] = (uint16_t)(p * S + s);
                                kcnt++;
                            }
                        }
                    }
                }
                if (kcnt > kKCap) brute = true;
            }
            if (!brute) {
                for (int i = 0; i < kcnt; i++) {
                    const int k = klist[i][tid];
                    const float sc = ref_score<D>(u, jh + (size_t)k * 4);
                    if (sc > bs || (sc == bs && k < bk)) { bs = sc; bk = k; }
                }
                idx = bk;
            }
        }
        if (brute) idx = brute_argmax<D>(u, jh, K);
        if (SPLIT) {
            // merge the slots: a slot that fell back to the exhaustive search holds the answer; otherwise the highest
            // exact score wins, the lowest index among equals; no candidate anywhere (all-zero direction) -> index 0
            float *bs_sh = reinterpret_cast<float *>(code_sh);
            int *bk_sh = reinterpret_cast<int *>(mask_sh);
            bs_sh[tid] = bs;
            bk_sh[tid] = brute ? (idx | (int)0x80000000) : (search ? bk : 0x7fffffff);
            __syncthreads();
            float ms = -INFINITY;
            int mk = 0x7fffffff;
            bool exact = false;
            for (int w = 0; w < slots; w++) {
                const int kw = bk_sh[w * n + c];
                const float sw = bs_sh[w * n + c];
                if (kw < 0) {
                    if (!exact) { exact = true; mk = kw & 0x7fffffff; }
                } else if (!exact && kw != 0x7fffffff && (sw > ms || (sw == ms && kw < mk))) {
                    ms = sw;
                    mk = kw;
                }
            }
            idx = mk == 0x7fffffff ? 0 : mk;
            __syncthreads();
        }
        if (a.stats && active) {
            if (brute && writer) atomicAdd(a.stats, 1);      // once per chunk, also when its slots split the search
            if (search && !brute) atomicAdd(a.stats + 1, cnt);
        }
    }

    // ---- per-token scale and radius code ----
    float rm = -INFINITY;
    bool rm_nan = false;
    if ((n & (n - 1)) == 0 && n <= 64) {
        // the n lanes of a token sit side by side inside one wavefront
        const int lane = tid & 63;
        const uint64_t tok_lanes = n == 64 ? ~0ull : ((1ull << n) - 1ull) << (lane / n * n);
        rm_nan = (__builtin_amdgcn_ballot_w64(is_nan(r)) & tok_lanes) != 0ull;
        rm = group_max(is_nan(r) ? -INFINITY : r, n, [](float p, float q) { return q > p ? q : p; });
    } else {
        const int base = tok_local * n;
        for (int i = 0; i < n; i++) {
            float o = (base + i < kQThreads) ? radius_sh[base + i] : 0.f;
            if (is_nan(o)) rm_nan = true;
            else if (o > rm) rm = o;
        }
    }
    rm = clamp_min_d<D>(rm_nan ? NAN : rm, 1e-8f);
    const float qmaxf = (float)a.qmax;
    const float scale = D::rnd(rm / qmaxf);
    float qf = rintf(D::rnd(r / scale));
    if (!is_nan(qf)) qf = fminf(fmaxf(qf, 0.f), qmaxf);
    const int rq = is_nan(qf) ? 0 : (int)qf;

    bool flagged = false;
    if (a.thr) flagged = nrm > D::load((const ST *)a.thr + h);

    if (active && writer) {
        const size_t o = (((size_t)b * a.H + h) * a.T + t) * n + c;
        if (a.idx_out) a.idx_out[o] = idx;
        if (a.rq_out) a.rq_out[o] = rq;
        if (a.mask_out) a.mask_out[o] = flagged ? 1 : 0;
        if (a.rmax_out && c == 0) D::store((ST *)a.rmax_out + o / n, rm);
        if (a.dense_out) {
            ST *dst = (ST *)a.dense_out + o * 4;
            if (flagged) {
                const ST *xp = (const ST *)a.x + b * a.xsb + h * a.xsh + (int64_t)t * a.xst + c * 4;
                for (int j = 0; j < 4; j++) dst[j] = xp[j];
            } else {
                const float rqs = D::rnd(qf * scale);
                const ST *row = jh + (size_t)idx * 4;
                for (int j = 0; j < 4; j++) D::store(dst + j, D::rnd(rqs * D::load(row + j)));
            }
        }
    }

    // ---- packed rows ----
    if (a.main_plane || a.flag_plane || a.scale_plane) {
        const int64_t row = (a.pos ? a.pos[b] : 0) + a.t_off + t;
        const bool row_ok = active && writer && row >= 0 && row < a.t_cap;  // a bad pos[] must not write outside the plane
        // Sideband compaction in the same launch, for appends whose new rows of a (b, h) all sit in this block
        // (T <= tokens_per_block; n a power of two, so the lanes of a token share a wavefront).  Entries, tile
        // offsets and counters come out as the in-order compaction kernel leaves them: flagged chunks in
        // (row, chunk) order behind the entries already there, the offset of a tile = the count before its
        // first row.  The entry slots are worked out before the rows are packed: a flagged chunk that finds the
        // sideband full is packed as a plain chunk (its radius code, no flag) instead of decoding to zero.
        bool keep = flagged;            // stays an outlier in the packed planes
        bool entry = false;             // this lane writes a sideband entry
        int ent_slot = 0, tile_first = 0, ent_total = 0;
        if (a.compact) {
            __syncthreads();            // radius_sh is free from here on
            const bool f = row_ok && flagged;
            const uint64_t m = __builtin_amdgcn_ballot_w64(f);
            const int lane = tid & 63;
            const uint64_t tok_bits = n == 64 ? ~0ull : ((1ull << n) - 1ull) << ((lane / n) * n);
            const int before_c = __popcll(m & tok_bits & ((1ull << lane) - 1ull));
            int *cnt_sh = reinterpret_cast<int *>(radius_sh);           // free since the scales were taken
            if (c == 0 && tok_local < a.tokens_per_block) cnt_sh[tok_local] = __popcll(m & tok_bits);
            const int base = a.sb_count[(size_t)b * a.H + h];           // read by every thread before the barrier,
            __syncthreads();                                            // rewritten by one thread at the end
            int mine = base, total = base;
            for (int i = 0; i < a.T; i++) {
                const int ci = cnt_sh[i];
                if (i < tok_local) mine += ci;
                total += ci;
            }
            tile_first = mine;
            ent_total = total;
            ent_slot = mine + before_c;
            entry = f && ent_slot < a.sb_cap;
            if (f && !entry) {
                keep = false;
                *a.overflow = 1;
            }
        }
        // a flagged chunk is read from the sideband; its packed code keeps idx with radius code 0, which decodes to zero
        code_sh[tid] = (uint32_t)idx | ((uint32_t)(keep ? 0 : rq) << a.idx_bits);
        mask_sh[tid] = keep ? 1u : 0u;
        __syncthreads();
        // one-bit planes (flags, a one-bit aux field) of tokens whose lanes sit side by side in a wavefront come
        // straight from a ballot: the token's n bits are n / 8 whole bytes of it
        const bool side_by_side = (n & (n - 1)) == 0 && n >= 8 && n <= 64;
        const int lane_base = (tid & 63) / n * n;
        const uint64_t aux_bits1 = __builtin_amdgcn_ballot_w64(((code_sh[tid] >> a.main_bits) & 1u) != 0u);
        const uint64_t flag_bits1 = __builtin_amdgcn_ballot_w64(keep);
        if (row_ok) {
            const size_t prow = ((size_t)b * a.H + h) * a.t_cap + row;
            const uint32_t *codes = code_sh + tok_local * n;
            if (a.main_plane) {
                const int rb = (n * a.main_bits + 7) >> 3;
                uint8_t *dst = a.main_plane + prow * rb;
                if (a.main_bits == 16) {
                    reinterpret_cast<uint16_t *>(dst)[c] = (uint16_t)codes[c];   // one code per lane
                } else if (a.main_bits == 12 && !(n & 1)) {
                    if (!(c & 1)) {                                             // two codes = three bytes
                        const uint32_t two = (codes[c] & 0xfffu) | ((codes[c + 1] & 0xfffu) << 12);
                        uint8_t *d = dst + (c >> 1) * 3;
                        d[0] = (uint8_t)two;
                        d[1] = (uint8_t)(two >> 8);
                        d[2] = (uint8_t)(two >> 16);
                    }
                } else {
                    for (int byte = c; byte < rb; byte += n) dst[byte] = gather_byte(codes, n, a.main_bits, 0, byte);
                }
            }
            if (a.aux_plane && a.aux_bits) {
                const int rb = (n * a.aux_bits + 7) >> 3;
                uint8_t *dst = a.aux_plane + prow * rb;
                if (a.aux_bits == 1 && side_by_side) {
                    if (c < rb) dst[c] = (uint8_t)(aux_bits1 >> (lane_base + 8 * c));
                } else {
                    for (int byte = c; byte < rb; byte += n) dst[byte] = gather_byte(codes, n, a.aux_bits, a.main_bits, byte);
                }
            }
            if (a.flag_plane) {
                const int rb = (n + 7) >> 3;
                uint8_t *dst = a.flag_plane + prow * rb;
                if (side_by_side) {
                    if (c < rb) dst[c] = (uint8_t)(flag_bits1 >> (lane_base + 8 * c));
                } else {
                    for (int byte = c; byte < rb; byte += n) dst[byte] = gather_byte(mask_sh + tok_local * n, n, 1, 0, byte);
                }
            }
            if (a.scale_plane && c == 0) D::store((ST *)a.scale_plane + prow, rm);
        }
        if (a.scale_max && a.scale_plane) {
            // the largest finite scale written so far, for the attention kernels' range guard: the wavefront's maximum,
            // and an atomic only when it raises the value (after the first blocks it hardly ever does)
            uint32_t mine = (row_ok && c == 0 && rm < INFINITY) ? __float_as_uint(rm) : 0u;     // scales are positive: bits order like values
            mine = group_max(mine, 64, [](uint32_t p, uint32_t q) { return max(p, q); });
            if ((tid & 63) == 0 && mine > __hip_atomic_load(a.scale_max, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                atomicMax(a.scale_max, mine);
        }
        if (a.compact) {
            const size_t bhs = (size_t)b * a.H + h;
            if (row_ok) {
                const int64_t tiles = (a.t_cap + kTile - 1) / kTile;
                if (c == 0 && (row & (kTile - 1)) == 0) a.sb_tile_off[bhs * tiles + (row >> 4)] = tile_first;
                if (entry) {
                    const ST *xp = (const ST *)a.x + b * a.xsb + h * a.xsh + (int64_t)t * a.xst + c * 4;
                    ST *dst = (ST *)a.sideband + (bhs * a.sb_cap + ent_slot) * 4;
                    for (int j = 0; j < 4; j++) dst[j] = xp[j];
                    if (a.sb_coord) a.sb_coord[bhs * a.sb_cap + ent_slot] = (uint16_t)(((row & (kTile - 1)) << 8) | c);
                }
            }
            if (tid == 0) a.sb_count[bhs] = ent_total;
        }
    }
}

template <class D, int ALGO>
__global__ __launch_bounds__(kQThreads) void quantize_kernel(QParams a) {
    quantize_body<D, ALGO>(a);
}

// The K and the V rows of one append in one launch (same shapes): blockIdx.z picks the tensor.  A single-token
// append is latency-bound (32 lanes per block for a few microseconds), so the two run side by side for free.
struct QPair {
    QParams p[2];       // K, V
};
// (indexed in the kernel-argument segment: one set of scalar registers, not a select per field of two structs)
template <class D, bool SPLIT>
__global__ __launch_bounds__(kQThreads) void quantize_pair_kernel(QPair kv) {
    quantize_body<D, 0, SPLIT>(kv.p[blockIdx.z]);
}
template <class D>
__global__ __launch_bounds__(kQThreads) void quantize_split_kernel(QParams a) {
    quantize_body<D, 0, true>(a);
}

// one new token per sequence, 16-bit dtype, the lanes of a token inside a wavefront: the split search
template <class D>
static bool use_split(const QParams &p, int algo) {
    return sizeof(typename D::storage) == 2 && algo == 0 && p.T == 1 && p.n >= 4 && p.n <= 64 && !(p.n & (p.n - 1));
}

template <class D>
static int launch_quantize(const QParams &p, int algo, hipStream_t st) {
    dim3 grid((p.T + p.tokens_per_block - 1) / p.tokens_per_block, p.B * p.H), block(kQThreads);
    size_t shmem = (size_t)p.S * 4 * sizeof(float) + (size_t)p.S * 4 * sizeof(uint2);
    if constexpr (sizeof(typename D::storage) == 2) {
        if (use_split<D>(p, algo)) {
            hipLaunchKernelGGL(quantize_split_kernel<D>, grid, block, shmem, st, p);
            return hip_status(hipGetLastError());
        }
    }
    if (algo == 1) hipLaunchKernelGGL((quantize_kernel<D, 1>), grid, block, shmem, st, p);
    else hipLaunchKernelGGL((quantize_kernel<D, 0>), grid, block, shmem, st, p);
    return hip_status(hipGetLastError());
}

template <class D>
static int launch_quantize_pair(const QParams &k, const QParams &v, hipStream_t st) {
    dim3 grid((k.T + k.tokens_per_block - 1) / k.tokens_per_block, k.B * k.H, 2), block(kQThreads);
    size_t shmem = (size_t)k.S * 4 * sizeof(float) + (size_t)k.S * 4 * sizeof(uint2);
    if constexpr (sizeof(typename D::storage) == 2) {
        if (use_split<D>(k, 0) && use_split<D>(v, 0)) {
            hipLaunchKernelGGL((quantize_pair_kernel<D, true>), grid, block, shmem, st, QPair{{k, v}});
            return hip_status(hipGetLastError());
        }
    }
    hipLaunchKernelGGL((quantize_pair_kernel<D, false>), grid, block, shmem, st, QPair{{k, v}});
    return hip_status(hipGetLastError());
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int hqmq_layout_bits(int S, int radius_bits, int *idx_bits, int *main_bits, int *aux_bits) {
    return layout_bits(S, radius_bits, idx_bits, main_bits, aux_bits);
}

// Checks one call's arguments and fills the kernel parameters; *empty is set for T == 0 (nothing to launch).
static int fill_qparams(const hqmq_quantize_args *a, QParams *out, bool *empty) {
    *empty = false;
    if (!a || !a->x || !a->joint) return HQMQ_ERR_NULL;
    if (a->algo == 0 && !a->slack) return HQMQ_ERR_NULL;
    if (a->B < 1 || a->H < 1 || a->T < 0 || a->n_chunks < 1 || a->n_chunks > kQThreads) return HQMQ_ERR_SHAPE;
    if ((int64_t)a->B * a->H > 65535) return HQMQ_ERR_SHAPE;
    if (a->T == 0) { *empty = true; return HQMQ_OK; }
    int ib, mb, ab;
    int rc = layout_bits(a->secondary_size, a->radius_bits, &ib, &mb, &ab);
    if (rc) return rc;
    if (24 * a->secondary_size > 65535) return HQMQ_ERR_SHAPE;  // candidate lists hold 16-bit indices
    const bool packed = a->main_plane || a->aux_plane || a->flag_plane || a->scale_plane;
    if (packed) {
        // the layout rule's widths, or any wider split that still holds idx_bits + radius_bits (16-bit rows for heads
        // whose lanes would otherwise get an odd number of 12-bit codes)
        if (a->main_bits < 1 || a->main_bits > 16 || a->aux_bits < 0 || a->aux_bits > 8 ||
            a->main_bits + a->aux_bits < ib + a->radius_bits)
            return HQMQ_ERR_LAYOUT;
        if (a->aux_bits && a->main_plane && !a->aux_plane) return HQMQ_ERR_NULL;
        if (a->t_cap < 1 || a->t_off < 0) return HQMQ_ERR_SHAPE;
        if (!a->pos && (int64_t)a->t_off + a->T > a->t_cap) return HQMQ_ERR_SHAPE;
        if (a->flag_plane && !a->thr) return HQMQ_ERR_NULL;
    }
    if (a->dtype != HQMQ_F32 && a->dtype != HQMQ_F16 && a->dtype != HQMQ_BF16) return HQMQ_ERR_DTYPE;
    QParams &p = *out;
    p.x = a->x; p.xsb = a->x_stride_b; p.xsh = a->x_stride_h; p.xst = a->x_stride_t;
    p.B = a->B; p.H = a->H; p.T = a->T; p.n = a->n_chunks;
    p.joint = a->joint; p.slack = a->slack; p.S = a->secondary_size; p.qmax = (1 << a->radius_bits) - 1;
    p.idx_out = a->idx_out; p.rq_out = a->rq_out; p.rmax_out = a->rmax_out; p.dense_out = a->dense_out;
    p.thr = a->thr; p.mask_out = a->mask_out;
    p.main_plane = a->main_plane; p.aux_plane = a->aux_plane; p.flag_plane = a->flag_plane;
    p.scale_plane = a->scale_plane; p.t_cap = a->t_cap; p.t_off = a->t_off; p.pos = a->pos;
    p.idx_bits = ib; p.main_bits = packed ? a->main_bits : mb; p.aux_bits = packed ? a->aux_bits : ab;
    p.tokens_per_block = kQThreads / a->n_chunks;
    p.stats = a->stats;
    p.scale_max = a->scale_max_bits;
    p.compact = 0;
    p.sideband = nullptr; p.sb_cap = 0; p.sb_tile_off = p.sb_count = p.overflow = nullptr; p.sb_coord = nullptr;
    return HQMQ_OK;
}

// The compaction of a short append can ride in the quantize launch: all new rows of a (b, h) in one block, the
// lanes of a token inside one wavefront, Med3x flags being written.
static bool take_compaction(QParams &p, const CompactCall *c) {
    if (!c || !p.thr || !p.flag_plane || p.T > p.tokens_per_block || (p.n & (p.n - 1)) || p.n > 64) return false;
    p.compact = 1;
    p.sideband = c->sideband; p.sb_cap = c->sb_cap; p.sb_tile_off = c->sb_tile_off; p.sb_count = c->sb_count;
    p.overflow = c->overflow; p.sb_coord = c->sb_coord;
    return true;
}

static int launch_one_tensor(const QParams &p, int dtype, int algo, hipStream_t st) {
    switch (dtype) {
        case HQMQ_F32: return launch_quantize<F32>(p, algo, st);
        case HQMQ_F16: return launch_quantize<F16>(p, algo, st);
        default: return launch_quantize<BF16>(p, algo, st);
    }
}

extern "C" int hqmq_quantize(const hqmq_quantize_args *a, void *stream) {
    QParams p;
    bool empty;
    const int rc = fill_qparams(a, &p, &empty);
    if (rc || empty) return rc;
    return launch_one_tensor(p, a->dtype, a->algo, (hipStream_t)stream);
}

int hqmq::quantize_two(const hqmq_quantize_args *k, const hqmq_quantize_args *v, const CompactCall *ck, const CompactCall *cv,
                       bool compacted[2], hipStream_t st) {
    QParams pk, pv;
    bool ek, ev;
    int rc = fill_qparams(k, &pk, &ek);
    if (rc) return rc;
    rc = fill_qparams(v, &pv, &ev);
    if (rc) return rc;
    compacted[0] = !ek && take_compaction(pk, ck);
    compacted[1] = !ev && take_compaction(pv, cv);
    const bool same = !ek && !ev && k->dtype == v->dtype && k->B == v->B && k->H == v->H && k->T == v->T &&
                      k->n_chunks == v->n_chunks && k->secondary_size == v->secondary_size && k->algo == 0 && v->algo == 0;
    if (same) {
        switch (k->dtype) {
            case HQMQ_F32: return launch_quantize_pair<F32>(pk, pv, st);
            case HQMQ_F16: return launch_quantize_pair<F16>(pk, pv, st);
            default: return launch_quantize_pair<BF16>(pk, pv, st);
        }
    }
    if (!ek) {
        rc = launch_one_tensor(pk, k->dtype, k->algo, st);
        if (rc) return rc;
    }
    return ev ? HQMQ_OK : launch_one_tensor(pv, v->dtype, v->algo, st);
}
