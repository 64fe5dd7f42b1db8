// Fused attention over the bit-packed HQMQ cache: decode (T_q = 1) and chunked prefill.
//
// Semantics follow fused_hqmq_attention_torch (src/quantizers/hqmq_attention.py:68-101 of
// the reference): K/V = codeword * (rq * rs / qmax), GQA broadcast, softmax(Q K^T * scale) V
// with SDPA's top-left causal alignment; it stands in for fused_hqmq_attention_triton (:425-518).
//
// Mapping (one wavefront = one work item = 16 query columns x one KV split):
//   * a "column" is a (query token, query head of the KV group) pair, so the G heads of a
//     GQA group - and several query tokens in prefill - share every decoded KV tile;
//   * scores are computed transposed, S^T = K_tile . Q^T, with v_mfma_f32_16x16x16_f16:
//     the A operand wants, per lane, 4 consecutive k-elements of one row - exactly one
//     decoded quaternion chunk of one token (row = token, k = 4 head dims);
//   * the S^T accumulator layout (lane = column + 16*(token/4), 4 tokens per lane) is the B
//     operand layout of the second MFMA, O^T = V^T . P^T, so P never leaves registers;
//   * V^T needs 4 tokens of one head dim per lane: each lane decodes one chunk (4 dims of
//     one token) and the four lanes of a quad transpose their 4x4 block with DPP moves;
//   * codewords come from a per-head fp16 copy of the joint table in LDS (8-byte gathers);
//   * KV is walked in super-tiles of 64 tokens; each lane reads its codes with one aligned
//     vector load per 16-token tile, a wavefront covering whole 128-byte lines of the plane;
//   * split-KV partials (m, l, acc) go to a workspace and are merged by a second kernel.
#include "common.h"

namespace hqmq {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kAttnWaves = 4;
constexpr int kSuper = 64;  // tokens per super-tile

struct PackedDev {
    const uint8_t *main_plane, *aux_plane, *flag_plane;
    const void *scale_plane;
    int64_t ssb, ssh, sst;
    const void *sideband;
    const int32_t *sb_tile_off;
    int64_t sb_cap;
    const void *joint;
    int64_t jsh;
    int K;
};

struct AttnParams {
    const void *Q;
    void *O;
    int64_t qsb, qsh, qst, osb, osh, ost;
    PackedDev Kc, Vc;
    int dtype;
    int B, Hq, Hkv, G, Tq, Tkv, n;
    int64_t t_cap;
    int idx_bits, aux_bits, qmax;
    const int32_t *kv_len;
    int causal;
    int64_t causal_offset;
    float c_log2;   // softmax_scale * log2(e) / qmax
    float c_plain;  // softmax_scale * log2(e)
    float inv_qmax;
    int n_splits, n_cg;
    float *ws;
};

__device__ __forceinline__ float load_any(const void *p, int dtype, int64_t i) {
    if (dtype == HQMQ_F16) return __half2float(__ushort_as_half(((const uint16_t *)p)[i]));
    if (dtype == HQMQ_BF16) return __uint_as_float((uint32_t)((const uint16_t *)p)[i] << 16);
    return ((const float *)p)[i];
}
__device__ __forceinline__ void store_any(void *p, int dtype, int64_t i, float f) {
    if (dtype == HQMQ_F16) ((uint16_t *)p)[i] = __half_as_ushort(__float2half_rn(f));
    else if (dtype == HQMQ_BF16) ((uint16_t *)p)[i] = f32_to_bf16_bits(f);
    else ((float *)p)[i] = f;
}
__device__ __forceinline__ half4 load_chunk_h(const void *p, int dtype, int64_t chunk) {
    half4 r;
    if (dtype == HQMQ_F16) {
        const uint2 w = *reinterpret_cast<const uint2 *>((const uint16_t *)p + chunk * 4);
        r = __builtin_bit_cast(half4, w);
    } else {
        for (int j = 0; j < 4; j++) r[j] = (_Float16)load_any(p, dtype, chunk * 4 + j);
    }
    return r;
}

// The lane's NB = CPL*MB/8 bytes of main-plane codes, as 32-bit words.
template <int NB>
__device__ __forceinline__ void load_bytes(const uint8_t *p, uint32_t (&w)[(NB + 3) / 4]) {
    constexpr int NW = (NB + 3) / 4;
    if constexpr (NB % 16 == 0) {
        for (int i = 0; i < NB / 16; i++) {
            const uint4 v = reinterpret_cast<const uint4 *>(p)[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
    } else if constexpr (NB % 8 == 0) {
        for (int i = 0; i < NB / 8; i++) {
            const uint2 v = reinterpret_cast<const uint2 *>(p)[i];
            w[2 * i] = v.x; w[2 * i + 1] = v.y;
        }
    } else if constexpr (NB % 4 == 0) {
        for (int i = 0; i < NW; i++) w[i] = reinterpret_cast<const uint32_t *>(p)[i];
    } else if constexpr (NB % 2 == 0) {
        for (int i = 0; i < NW; i++) w[i] = 0;
        for (int i = 0; i < NB / 2; i++) w[i >> 1] |= (uint32_t) reinterpret_cast<const uint16_t *>(p)[i] << (16 * (i & 1));
    } else {
        for (int i = 0; i < NW; i++) w[i] = 0;
        for (int i = 0; i < NB; i++) w[i >> 2] |= (uint32_t)p[i] << (8 * (i & 3));
    }
}

template <int MB, int NW>
__device__ __forceinline__ uint32_t code_at(const uint32_t (&w)[NW], int j) {
    const int pos = j * MB, wd = pos >> 5, sh = pos & 31;
    uint32_t v = w[wd] >> sh;
    if (sh + MB > 32 && wd + 1 < NW) v |= w[wd + 1] << (32 - sh);
    return v & ((1u << MB) - 1u);
}

// aux bits of the lane's CPL codes: bits [first_code*ab, (first_code+CPL)*ab) of the aux row
template <int CPL>
__device__ __forceinline__ uint64_t load_aux(const uint8_t *row, int row_bytes, int first_code, int ab) {
    const int start = first_code * ab, nbits = CPL * ab;
    const int b0 = start >> 3, sh = start & 7;
    uint64_t v = 0;
    for (int i = 0; i * 8 < nbits + sh && b0 + i < row_bytes && i < 8; i++) v |= (uint64_t)row[b0 + i] << (8 * i);
    v >>= sh;
    if (nbits + sh > 64 && b0 + 8 < row_bytes) v |= (uint64_t)row[b0 + 8] << (64 - sh);
    return v;
}

__device__ __forceinline__ uint32_t dpp_quad_xor2(uint32_t v) {  // lane i <- lane i^2 within each quad
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
}
__device__ __forceinline__ uint32_t dpp_quad_xor1(uint32_t v) {  // lane i <- lane i^1
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
}

// Quad lane i holds (e(i,0), e(i,1)) in r0 and (e(i,2), e(i,3)) in r1; afterwards lane i holds
// (e(0,i), e(1,i)) in r0 and (e(2,i), e(3,i)) in r1.
__device__ __forceinline__ void quad_transpose(uint32_t &r0, uint32_t &r1, int lane) {
    const bool upper = lane & 2;
    const uint32_t send = upper ? r0 : r1;
    const uint32_t recv = dpp_quad_xor2(send);
    const uint32_t X = upper ? recv : r0, Y = upper ? r1 : recv;
    const uint32_t PX = dpp_quad_xor1(X), PY = dpp_quad_xor1(Y);
    const uint32_t sel = (lane & 1) ? 0x03020706u : 0x05040100u;
    r0 = __builtin_amdgcn_perm(PX, X, sel);
    r1 = __builtin_amdgcn_perm(PY, Y, sel);
}


// Flag bookkeeping for one 16-token tile. Every lane passes the token it decodes (`tok`, 0..15)
// and the first chunk of its code group; returns the lane's CPL flag bits and the sideband slot
// of its first flagged chunk: tile offset + flagged chunks of earlier tokens + earlier chunks.
template <int CPL>
__device__ __forceinline__ void tile_flags(const PackedDev &c, size_t plane_row0, int64_t tile_row, int64_t t_cap, int frb,
                                           size_t tile_off_index, int col, int tok, int first, uint32_t &fl, int &slot0) {
    int64_t row = tile_row + col;
    if (row >= t_cap) row = t_cap - 1;
    uint32_t fw = 0;
    const uint8_t *fr = c.flag_plane + (plane_row0 + row) * frb;
    for (int i = 0; i < frb && i < 4; i++) fw |= (uint32_t)fr[i] << (8 * i);
    const int own = __popc(fw);
    int pre = own;
    for (int o = 1; o < 16; o <<= 1) {
        const int v = __shfl_up(pre, o, 16);
        if (col >= o) pre += v;
    }
    pre -= own;                          // flagged chunks in tokens < col of this tile
    const uint32_t fw_t = (uint32_t)__shfl((int)fw, tok, 16);
    const int pre_t = __shfl(pre, tok, 16);
    fl = (fw_t >> first) & ((CPL >= 32) ? 0xffffffffu : ((1u << CPL) - 1u));
    slot0 = c.sb_tile_off[tile_off_index] + pre_t + __popc(fw_t & ((first >= 32) ? 0xffffffffu : ((1u << first) - 1u)));
}

// A flagged chunk: the verbatim values from the sideband (exact in fp16 for fp16 caches).
__device__ __forceinline__ half4 outlier_chunk(const PackedDev &c, int dtype, size_t bh, int slot) {
    int64_t s = slot;
    if (s >= c.sb_cap) s = c.sb_cap - 1;
    return load_chunk_h(c.sideband, dtype, (int64_t)bh * c.sb_cap + s);
}

template <int CPL, int MB, bool FLAGS>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_kernel(AttnParams p) {
    constexpr int NB = CPL * MB / 8;
    constexpr int NW = (NB + 3) / 4;
    extern __shared__ uint2 lds_tab[];
    uint2 *ktab = lds_tab, *vtab = lds_tab + p.Kc.K;

    const int bh = blockIdx.y, b = bh / p.Hkv, hkv = bh - b * p.Hkv;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int dtype = p.dtype;

    // ---- per-head codeword tables -> LDS as fp16 ----
    for (int k = threadIdx.x; k < p.Kc.K; k += blockDim.x)
        ktab[k] = __builtin_bit_cast(uint2, load_chunk_h(p.Kc.joint, dtype, hkv * (p.Kc.jsh / 4) + k));
    for (int k = threadIdx.x; k < p.Vc.K; k += blockDim.x)
        vtab[k] = __builtin_bit_cast(uint2, load_chunk_h(p.Vc.joint, dtype, hkv * (p.Vc.jsh / 4) + k));
    __syncthreads();

    const int item = blockIdx.x * kAttnWaves + wave;
    if (item >= p.n_cg * p.n_splits) return;
    const int cg = item / p.n_splits, sp = item - cg * p.n_splits;

    const int n = p.n, G = p.G;
    const int col = lane & 15, grp = lane >> 4;
    const int cidx = cg * 16 + col;
    const bool col_ok = cidx < p.Tq * G;
    const int tq = col_ok ? cidx / G : 0, g = col_ok ? cidx - tq * G : 0;
    const int hq = hkv * G + g;

    // ---- Q^T fragment: lane (col, grp) holds dims [grp*CPL*4, +CPL*4) of its column ----
    half4 qf[CPL];
    {
        const int64_t base = b * p.qsb + hq * p.qsh + (int64_t)tq * p.qst + grp * CPL * 4;
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            if (col_ok) qf[j] = load_chunk_h((const char *)p.Q + base * (dtype == HQMQ_F32 ? 4 : 2), dtype, j);
            else qf[j] = half4{0, 0, 0, 0};
        }
    }

    // ---- KV range of this item ----
    int kv_end = p.kv_len ? p.kv_len[b] : p.Tkv;
    if (kv_end > p.Tkv) kv_end = p.Tkv;
    if (kv_end < 0) kv_end = 0;
    // per-column visible limit (exclusive)
    int64_t lim64 = kv_end;
    if (p.causal) {
        const int64_t cl = (int64_t)tq + p.causal_offset + 1;
        if (cl < lim64) lim64 = cl;
    }
    if (!col_ok || lim64 < 0) lim64 = 0;
    const int col_lim = (int)lim64;
    // wave-wide limit: max over the 16 columns (columns are ordered by query token)
    int wave_lim = col_lim;
    for (int o = 1; o < 16; o <<= 1) wave_lim = max(wave_lim, __shfl_xor(wave_lim, o));
    int per_split = (wave_lim + p.n_splits - 1) / p.n_splits;
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int t_begin = sp * per_split;
    const int t_end = min(wave_lim, t_begin + per_split);

    const size_t plane_row0 = (size_t)bh * p.t_cap;
    const int mrb = n * MB / 8;
    const int arb = (n * p.aux_bits + 7) >> 3;
    const int frb = (n + 7) >> 3;
    const int64_t tiles_cap = (p.t_cap + kTile - 1) / kTile;
    const uint32_t idx_mask = (1u << p.idx_bits) - 1u;
    const int idx_bits = p.idx_bits, ab = p.aux_bits;

    float m_run = -INFINITY, l_run = 0.f;
    float4v acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};

    // K-side lane role: token = col (row of the A operand), code group = grp
    // V-side lane role: token = 4*grp + (col & 3), code group = col >> 2
    const int v_tok = 4 * grp + (col & 3), v_grp = col >> 2;

    for (int t0 = t_begin; t0 < t_end; t0 += kSuper) {
        float4v sT[4], sTo[4];
        // ---------------- S^T = K . Q^T for 4 tiles ----------------
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int64_t row = (int64_t)t0 + 16 * u + col;
            if (row >= p.t_cap) row = p.t_cap - 1;
            uint32_t w[NW];
            load_bytes<NB>(p.Kc.main_plane + (plane_row0 + row) * mrb + grp * NB, w);
            uint64_t aux = 0;
            if (ab) aux = load_aux<CPL>(p.Kc.aux_plane + (plane_row0 + row) * arb, arb, grp * CPL, ab);
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Kc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, col, grp * CPL, fl, sb_base);
            float4v s = float4v{0.f, 0.f, 0.f, 0.f}, so = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                uint32_t code = code_at<MB, NW>(w, j);
                if (ab) code |= (uint32_t)((aux >> (j * ab)) & ((1u << ab) - 1u)) << MB;
                const uint32_t k = code & idx_mask;
                const _Float16 rq = (_Float16)(float)(code >> idx_bits);
                half4 a = __builtin_bit_cast(half4, ktab[k]);
                a = a * rq;
                if (FLAGS) {
                    // flagged chunks carry no rs/qmax factor: they go through their own accumulator
                    const bool f = (fl >> j) & 1u;
                    if (__builtin_amdgcn_ballot_w64(f) != 0) {
                        half4 ao = half4{0, 0, 0, 0};
                        if (f) {
                            ao = outlier_chunk(p.Kc, dtype, bh, sb_base + __popc(fl & ((1u << j) - 1u)));
                            a = half4{0, 0, 0, 0};
                        }
                        so = __builtin_amdgcn_mfma_f32_16x16x16f16(ao, qf[j], so, 0, 0, 0);
                    }
                }
                s = __builtin_amdgcn_mfma_f32_16x16x16f16(a, qf[j], s, 0, 0, 0);
            }
            sT[u] = s;
            if (FLAGS) sTo[u] = so;
        }
        // ---------------- scale, mask, online softmax ----------------
        float pv[4][4];
        float tmax = -INFINITY;
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int t = t0 + 16 * u + 4 * grp + e;
                float rs = 0.f;
                if (t < p.Tkv) rs = load_any(p.Kc.scale_plane, dtype, b * p.Kc.ssb + hkv * p.Kc.ssh + (int64_t)t * p.Kc.sst);
                float v = sT[u][e] * (rs * p.c_log2);
                if (FLAGS) v = fmaf(sTo[u][e], p.c_plain, v);
                v = (t < col_lim && t < t_end) ? v : -INFINITY;
                pv[u][e] = v;
                tmax = fmaxf(tmax, v);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = exp2f(m_run - m_use);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int j = 0; j < CPL; j++) acc[j] = acc[j] * alpha;
        half4 pT[4], pTo[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float pe = exp2f(pv[u][e] - m_use);
                l_run += pe;
                const int t = t0 + 16 * u + 4 * grp + e;
                float rs = 0.f;
                if (t < p.Tkv) rs = load_any(p.Vc.scale_plane, dtype, b * p.Vc.ssb + hkv * p.Vc.ssh + (int64_t)t * p.Vc.sst);
                pT[u][e] = (_Float16)(pe * (rs * p.inv_qmax));
                if (FLAGS) pTo[u][e] = (_Float16)pe;
                pv[u][e] = pe;
            }
        }
        // ---------------- O^T += V^T . P^T ----------------
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int64_t row = (int64_t)t0 + 16 * u + v_tok;
            if (row >= p.t_cap) row = p.t_cap - 1;
            uint32_t w[NW];
            load_bytes<NB>(p.Vc.main_plane + (plane_row0 + row) * mrb + v_grp * NB, w);
            uint64_t aux = 0;
            if (ab) aux = load_aux<CPL>(p.Vc.aux_plane + (plane_row0 + row) * arb, arb, v_grp * CPL, ab);
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Vc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, v_tok, v_grp * CPL, fl, sb_base);
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                uint32_t code = code_at<MB, NW>(w, j);
                if (ab) code |= (uint32_t)((aux >> (j * ab)) & ((1u << ab) - 1u)) << MB;
                const uint32_t k = code & idx_mask;
                const _Float16 rq = (_Float16)(float)(code >> idx_bits);
                half4 a = __builtin_bit_cast(half4, vtab[k]);
                a = a * rq;
                if (FLAGS) {
                    const bool f = (fl >> j) & 1u;
                    if (__builtin_amdgcn_ballot_w64(f) != 0) {
                        half4 ao = half4{0, 0, 0, 0};
                        if (f) {
                            ao = outlier_chunk(p.Vc, dtype, bh, sb_base + __popc(fl & ((1u << j) - 1u)));
                            a = half4{0, 0, 0, 0};
                        }
                        uint2 ro = __builtin_bit_cast(uint2, ao);
                        quad_transpose(ro.x, ro.y, lane);
                        acc[j] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, ro), pTo[u], acc[j], 0, 0, 0);
                    }
                }
                uint2 r = __builtin_bit_cast(uint2, a);
                quad_transpose(r.x, r.y, lane);
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, r), pT[u], acc[j], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: lane (col, grp) holds, for block j, dims 4*(CPL*grp + j) + 0..3 of column col ----
    float l_tot = l_run;
    l_tot += __shfl_xor(l_tot, 16);
    l_tot += __shfl_xor(l_tot, 32);
    if (!col_ok) return;
    if (p.n_splits == 1) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const int64_t base = b * p.osb + hq * p.osh + (int64_t)tq * p.ost + grp * CPL * 4;
#pragma unroll
        for (int j = 0; j < CPL; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) store_any(p.O, dtype, base + 4 * j + e, acc[j][e] * inv);
    } else {
        const int d_h = 4 * n;
        float *wp = p.ws + ((((size_t)b * p.Hq + hq) * p.Tq + tq) * p.n_splits + sp) * (size_t)(d_h + 2);
        if (grp == 0) { wp[0] = m_run; wp[1] = l_tot; }
#pragma unroll
        for (int j = 0; j < CPL; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) wp[2 + grp * CPL * 4 + 4 * j + e] = acc[j][e];
    }
}

// One thread per output element; merges the split partials of its row.
__global__ void attn_combine_kernel(const float *ws, void *O, int dtype, int B, int Hq, int Tq, int d_h, int n_splits,
                                    int64_t osb, int64_t osh, int64_t ost) {
    const int64_t total = (int64_t)B * Hq * Tq * d_h;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int e = (int)(g % d_h);
        const int64_t row = g / d_h;
        const int tq = (int)(row % Tq), hq = (int)((row / Tq) % Hq), b = (int)(row / ((int64_t)Tq * Hq));
        const float *wp = ws + (size_t)row * n_splits * (d_h + 2);
        float m = -INFINITY;
        for (int s = 0; s < n_splits; s++) m = fmaxf(m, wp[(size_t)s * (d_h + 2)]);
        float l = 0.f, o = 0.f;
        if (m > -INFINITY) {
            for (int s = 0; s < n_splits; s++) {
                const float *q = wp + (size_t)s * (d_h + 2);
                const float w = exp2f(q[0] - m);
                l += q[1] * w;
                o += q[2 + e] * w;
            }
        }
        store_any(O, dtype, b * osb + hq * osh + (int64_t)tq * ost + e, l > 0.f ? o / l : 0.f);
    }
}

static PackedDev to_dev(const hqmq_packed &k) {
    return PackedDev{k.main_plane, k.aux_plane, k.flag_plane, k.scale_plane, k.scale_sb, k.scale_sh, k.scale_st,
                     k.sideband, k.sb_tile_off, k.sb_cap, k.joint, k.joint_sh, k.K};
}

template <int CPL, int MB>
static int launch_attn(const AttnParams &p, bool flags, dim3 grid, size_t shmem, hipStream_t st) {
    auto kern = flags ? attn_kernel<CPL, MB, true> : attn_kernel<CPL, MB, false>;
    if (shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(kern, grid, dim3(kAttnWaves * 64), shmem, st, p);
    return hip_status(hipGetLastError());
}

template <int CPL>
static int launch_attn_mb(const AttnParams &p, int mb, bool flags, dim3 grid, size_t shmem, hipStream_t st) {
    switch (mb) {
        case 8: return launch_attn<CPL, 8>(p, flags, grid, shmem, st);
        case 12:
            if constexpr (CPL % 2 == 0) return launch_attn<CPL, 12>(p, flags, grid, shmem, st);
            else return HQMQ_ERR_SHAPE;
        case 16: return launch_attn<CPL, 16>(p, flags, grid, shmem, st);
        default: return HQMQ_ERR_LAYOUT;
    }
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int64_t hqmq_attn_workspace_bytes(int B, int H_q, int T_q, int d_h, int n_splits) {
    if (n_splits <= 1) return 0;
    return (int64_t)B * H_q * T_q * n_splits * (d_h + 2) * 4;
}

extern "C" int hqmq_attn_pick_splits(int B, int H_q, int H_kv, int T_q, int T_kv) {
    if (B < 1 || H_q < 1 || H_kv < 1 || T_q < 1 || T_kv < 1) return 1;
    const int G = H_q / H_kv;
    const int64_t base = (int64_t)B * H_kv * ((T_q * G + 15) / 16);
    int64_t s = (2048 + base - 1) / base;
    const int64_t cap = (T_kv + 2 * kSuper - 1) / (2 * kSuper);
    if (s > cap) s = cap;
    if (s < 1) s = 1;
    if (s > 512) s = 512;
    return (int)s;
}

extern "C" int hqmq_attn_fwd(const hqmq_attn_args *a, void *stream) {
    if (!a || !a->Q || !a->O) return HQMQ_ERR_NULL;
    const hqmq_packed *pk[2] = {&a->K, &a->V};
    for (const hqmq_packed *k : pk) {
        if (!k->main_plane || !k->scale_plane || !k->joint) return HQMQ_ERR_NULL;
        if (a->aux_bits && !k->aux_plane) return HQMQ_ERR_NULL;
        if (k->flag_plane && (!k->sideband || !k->sb_tile_off || k->sb_cap < 1)) return HQMQ_ERR_NULL;
        if (k->K < 1 || k->K > (1 << a->idx_bits) || (k->joint_sh & 3)) return HQMQ_ERR_SHAPE;
    }
    if (a->dtype != HQMQ_F32 && a->dtype != HQMQ_F16 && a->dtype != HQMQ_BF16) return HQMQ_ERR_DTYPE;
    if (a->B < 1 || a->H_q < 1 || a->H_kv < 1 || a->H_q % a->H_kv || a->T_q < 1 || a->T_kv < 0) return HQMQ_ERR_SHAPE;
    if ((int64_t)a->B * a->H_kv > 65535) return HQMQ_ERR_SHAPE;
    if (a->t_cap < a->T_kv || a->t_cap < 1) return HQMQ_ERR_SHAPE;
    const int n = a->n_chunks;
    if (n < 4 || n > 64 || (n & (n - 1)) || a->qmax < 1) return HQMQ_ERR_SHAPE;  // d_h in {16, 32, 64, 128, 256}
    if (a->idx_bits < 1 || a->idx_bits > 16 || a->aux_bits < 0 || a->aux_bits > 8) return HQMQ_ERR_LAYOUT;
    if ((a->K.flag_plane != nullptr) != (a->V.flag_plane != nullptr)) return HQMQ_ERR_NULL;
    const bool flags = a->K.flag_plane != nullptr;
    if (flags && n > 32) return HQMQ_ERR_SHAPE;
    const int elt = a->dtype == HQMQ_F32 ? 4 : 2;
    if (((uintptr_t)a->Q % (4 * elt)) || (a->q_sb % 4) || (a->q_sh % 4) || (a->q_st % 4)) return HQMQ_ERR_ALIGN;
    if (((uintptr_t)a->K.joint % (4 * elt)) || ((uintptr_t)a->V.joint % (4 * elt))) return HQMQ_ERR_ALIGN;
    if (((uintptr_t)a->K.main_plane & 15) || ((uintptr_t)a->V.main_plane & 15)) return HQMQ_ERR_ALIGN;
    if (flags && (((uintptr_t)a->K.sideband % (4 * elt)) || ((uintptr_t)a->V.sideband % (4 * elt)))) return HQMQ_ERR_ALIGN;

    int n_splits = a->n_splits > 0 ? a->n_splits : hqmq_attn_pick_splits(a->B, a->H_q, a->H_kv, a->T_q, a->T_kv);
    if (n_splits > 1) {
        if (!a->workspace) return HQMQ_ERR_NULL;
        if (a->workspace_bytes < hqmq_attn_workspace_bytes(a->B, a->H_q, a->T_q, 4 * n, n_splits)) return HQMQ_ERR_WORKSPACE;
        if ((uintptr_t)a->workspace & 3) return HQMQ_ERR_ALIGN;
    }
    const size_t shmem = ((size_t)a->K.K + a->V.K) * 8;
    if (shmem > 152 * 1024) return HQMQ_ERR_SHAPE;

    AttnParams p;
    p.Q = a->Q; p.O = a->O;
    p.qsb = a->q_sb; p.qsh = a->q_sh; p.qst = a->q_st; p.osb = a->o_sb; p.osh = a->o_sh; p.ost = a->o_st;
    p.Kc = to_dev(a->K); p.Vc = to_dev(a->V);
    p.dtype = a->dtype;
    p.B = a->B; p.Hq = a->H_q; p.Hkv = a->H_kv; p.G = a->H_q / a->H_kv; p.Tq = a->T_q; p.Tkv = a->T_kv; p.n = n;
    p.t_cap = a->t_cap;
    p.idx_bits = a->idx_bits; p.aux_bits = a->aux_bits; p.qmax = a->qmax;
    p.kv_len = a->kv_len; p.causal = a->causal; p.causal_offset = a->causal_offset;
    p.c_log2 = a->softmax_scale * 1.4426950408889634f / (float)a->qmax;
    p.c_plain = a->softmax_scale * 1.4426950408889634f;
    p.inv_qmax = 1.0f / (float)a->qmax;
    p.n_splits = n_splits;
    p.n_cg = (a->T_q * p.G + 15) / 16;
    p.ws = (float *)a->workspace;
    const int64_t items = (int64_t)p.n_cg * n_splits;
    dim3 grid((unsigned)((items + kAttnWaves - 1) / kAttnWaves), (unsigned)(a->B * a->H_kv));
    hipStream_t st = (hipStream_t)stream;
    int rc;
    switch (n / 4) {
        case 1: rc = launch_attn_mb<1>(p, a->main_bits, flags, grid, shmem, st); break;
        case 2: rc = launch_attn_mb<2>(p, a->main_bits, flags, grid, shmem, st); break;
        case 4: rc = launch_attn_mb<4>(p, a->main_bits, flags, grid, shmem, st); break;
        case 8: rc = launch_attn_mb<8>(p, a->main_bits, flags, grid, shmem, st); break;
        case 16: rc = launch_attn_mb<16>(p, a->main_bits, flags, grid, shmem, st); break;
        default: return HQMQ_ERR_SHAPE;
    }
    if (rc) return rc;
    if (n_splits > 1) {
        const int64_t total = (int64_t)a->B * a->H_q * a->T_q * 4 * n;
        int64_t g = (total + 255) / 256;
        if (g > 1 << 20) g = 1 << 20;
        hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)g), dim3(256), 0, st, (const float *)a->workspace, a->O,
                           a->dtype, a->B, a->H_q, a->T_q, 4 * n, n_splits, a->o_sb, a->o_sh, a->o_st);
        rc = hip_status(hipGetLastError());
    }
    return rc;
}
