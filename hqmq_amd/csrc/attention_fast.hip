// Attention kernels specialised at compile time for the layouts the BASELINE shapes use:
// d_h = 64 / 128, fp16 or bf16 caches, codes of 16+0 (s96_r4), 12+1 (s24_r3) or 16+3 (s192_r6) bits.
// Same algorithm and lane mapping as the generic kernel in attention.hip (see the notes there); what
// differs is that the dtype, the code widths and the aux width are template constants, the scales are
// kept as raw 16-bit words until use, and the register budget is held to two wavefronts per SIMD so that
// LDS gathers and MFMA latencies of one wavefront hide behind the other.
#include "attention_common.h"

namespace hqmq {

template <int DT>
__device__ __forceinline__ float cvt16(uint32_t bits16) {
    if (DT == HQMQ_F16) return __half2float(__ushort_as_half((uint16_t)bits16));
    return __uint_as_float(bits16 << 16);
}
template <int DT>
__device__ __forceinline__ half4 chunk_to_half(uint2 w) {
    if (DT == HQMQ_F16) return __builtin_bit_cast(half4, w);
    half4 r;
    r[0] = (_Float16)__uint_as_float(w.x << 16); r[1] = (_Float16)__uint_as_float(w.x & 0xffff0000u);
    r[2] = (_Float16)__uint_as_float(w.y << 16); r[3] = (_Float16)__uint_as_float(w.y & 0xffff0000u);
    return r;
}

// Both per-head tables -> LDS as fp16; every load of the block is in flight before the first store.
template <int DT, int NT>
__device__ __forceinline__ void fill_tables16(uint2 *kdst, const uint2 *ksrc, int Kk, uint2 *vdst, const uint2 *vsrc, int Kv) {
    constexpr int U = 5;
    for (int k0 = threadIdx.x; k0 < max(Kk, Kv); k0 += NT * U) {
        uint2 tk[U], tv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * NT;
            tk[u] = k < Kk ? ksrc[k] : uint2{0, 0};
            tv[u] = k < Kv ? vsrc[k] : uint2{0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * NT;
            if (k < Kk) kdst[k] = __builtin_bit_cast(uint2, chunk_to_half<DT>(tk[u]));
            if (k < Kv) vdst[k] = __builtin_bit_cast(uint2, chunk_to_half<DT>(tv[u]));
        }
    }
}

constexpr int kFastWaves = 8;

// codes, aux bits and raw 16-bit scales of one 64-token super-tile for one lane
template <int NW, int AB>
struct FastTile {
    uint32_t kw[4][NW], vw[4][NW];
    uint32_t kaux[AB ? 4 : 1], vaux[AB ? 4 : 1];
    uint2 ks[4], vs[4];
};

template <int NBYTES>
__device__ __forceinline__ uint32_t load_small(const uint8_t *p) {
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < NBYTES; i++) v |= (uint32_t)p[i] << (8 * i);
    return v;
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// two 16-bit scales (raw bits of dtype DT) as fp32 / as a packed fp16 pair
template <int DT>
__device__ __forceinline__ float scale_f32(uint32_t pair, int hi) {
    if (DT == HQMQ_F16) return (float)__builtin_bit_cast(half2v, pair)[hi];
    return __uint_as_float(hi ? (pair & 0xffff0000u) : (pair << 16));
}
template <int DT>
__device__ __forceinline__ half2v scale_h2(uint32_t pair) {
    if (DT == HQMQ_F16) return __builtin_bit_cast(half2v, pair);
    half2v r;
    r[0] = (_Float16)__uint_as_float(pair << 16);
    r[1] = (_Float16)__uint_as_float(pair & 0xffff0000u);
    return r;
}

// The V table sits at a fixed LDS offset so that its gathers use the instruction's immediate offset.
constexpr int kVTabOffset = 40960;          // bytes; room for 5120 K codewords in front of it

// Decodes the CPL chunks of one lane: gather from the LDS table (byte offset `tab`), times the radius code.
// 16+0 layout: the two radius codes of a dword become an fp16 pair with one shift, one and-or
// (0x6400 | rq is the fp16 number 1024 + rq) and one packed subtract; the two table addresses take a
// shift and a mask each.  IB = idx_bits when known at compile time (12 for s96), else 0.
template <int CPL, int MB, int AB, int IB, int NW>
__device__ __forceinline__ void decode_chunks(const uint32_t (&w)[NW], uint32_t aux, const char *tab, int idx_bits_rt,
                                              half4 (&a)[CPL]) {
    const int idx_bits = IB ? IB : idx_bits_rt;
    const uint32_t idx_mask = (1u << idx_bits) - 1u;
    if constexpr (MB == 16 && AB == 0) {
        const uint32_t rq2 = (0xffffu >> idx_bits) * 0x00010001u;
        const uint2 *t2 = reinterpret_cast<const uint2 *>(tab);
#pragma unroll
        for (int i = 0; i < CPL / 2; i++) {
            const uint32_t lo = w[i] & idx_mask, hi = (w[i] >> 16) & idx_mask;      // and / bit-field extract
            const uint32_t t = ((w[i] >> idx_bits) & rq2) | 0x64006400u;
            const half2v r = __builtin_bit_cast(half2v, t) - half2v{(_Float16)1024.0f, (_Float16)1024.0f};
            a[2 * i] = __builtin_bit_cast(half4, t2[lo]) * r[0];
            a[2 * i + 1] = __builtin_bit_cast(half4, t2[hi]) * r[1];
        }
    } else {
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            uint32_t code = code_at<MB, NW>(w, j);
            if (AB) code |= ((aux >> (j * AB)) & ((1u << AB) - 1u)) << MB;
            const _Float16 rq = (_Float16)(uint16_t)(code >> idx_bits);
            a[j] = __builtin_bit_cast(half4, reinterpret_cast<const uint2 *>(tab)[code & idx_mask]) * rq;
        }
    }
}

template <int CPL, int MB, int AB, int IB, int DT, bool FLAGS>
__global__ __launch_bounds__(kFastWaves * 64, 2) void attn_fast_kernel(AttnParams p) {
    constexpr int NB = CPL * MB / 8;
    constexpr int NW = (NB + 3) / 4;
    constexpr int ABYTES = CPL * AB / 8;     // aux bytes per lane (CPL * AB is a multiple of 8 here)
    static_assert(AB == 0 || (CPL * AB) % 8 == 0, "aux bits of one lane must be whole bytes");
    constexpr int NT = kFastWaves * 64;
    extern __shared__ uint2 lds_tab[];
    uint2 *ktab = lds_tab, *vtab = lds_tab + kVTabOffset / 8;
    const char *ktab_b = reinterpret_cast<const char *>(lds_tab), *vtab_b = ktab_b + kVTabOffset;

    const int bh = blockIdx.z, b = bh / p.Hkv, hkv = bh - b * p.Hkv;
    const int cg = blockIdx.y, sp = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int G = p.G;
    constexpr int n = 4 * CPL, d_h = 16 * CPL;
    const int col = lane & 15, grp = lane >> 4;
    const int cidx = cg * 16 + col;
    const bool col_ok = cidx < p.Tq * G;
    const int tq = col_ok ? cidx / G : 0, g = col_ok ? cidx - tq * G : 0;
    const int hq = hkv * G + g;

    int kv_end = p.kv_len ? p.kv_len[b] : p.Tkv;
    kv_end = min(max(kv_end, 0), p.Tkv);
    int64_t lim64 = kv_end;
    if (p.causal) lim64 = min(lim64, (int64_t)tq + p.causal_offset + 1);
    if (!col_ok || lim64 < 0) lim64 = 0;
    const int col_lim = (int)lim64;
    int blk_lim = col_lim, lim_min = col_ok ? col_lim : 0x7fffffff;
    for (int o = 1; o < 16; o <<= 1) {
        blk_lim = max(blk_lim, __shfl_xor(blk_lim, o));
        lim_min = min(lim_min, __shfl_xor(lim_min, o));
    }
    int per_split = (blk_lim + p.n_splits - 1) / p.n_splits;
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int b_begin = min(sp * per_split, blk_lim), b_end = min(blk_lim, b_begin + per_split);
    int per_wave = (b_end - b_begin + kFastWaves - 1) / kFastWaves;
    per_wave = (per_wave + kSuper - 1) / kSuper * kSuper;
    const int t_begin = min(b_begin + wave * per_wave, b_end), t_end = min(b_end, t_begin + per_wave);

    const size_t plane_row0 = (size_t)bh * p.t_cap;
    constexpr int mrb = n * MB / 8, arb = (n * AB + 7) / 8, frb = (n + 7) / 8;
    const int64_t tiles_cap = (p.t_cap + kTile - 1) / kTile;
    const int idx_bits = p.idx_bits;
    const int v_tok = 4 * grp + (col & 3), v_grp = col >> 2;
    const uint16_t *ks_plane = (const uint16_t *)p.Kc.scale_plane + b * p.Kc.ssb + hkv * p.Kc.ssh;
    const uint16_t *vs_plane = (const uint16_t *)p.Vc.scale_plane + b * p.Vc.ssb + hkv * p.Vc.ssh;
    const uint8_t *k_rows = p.Kc.main_plane + plane_row0 * mrb + grp * NB;
    const uint8_t *v_rows = p.Vc.main_plane + plane_row0 * mrb + v_grp * NB;
    const uint8_t *ka_rows = AB ? p.Kc.aux_plane + plane_row0 * arb + grp * ABYTES : nullptr;
    const uint8_t *va_rows = AB ? p.Vc.aux_plane + plane_row0 * arb + v_grp * ABYTES : nullptr;
    const int64_t last_row = p.t_cap - 1;

    auto load_super = [&](int t0, FastTile<NW, AB> &s) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int64_t krow = min((int64_t)t0 + 16 * u + col, last_row);
            const int64_t vrow = min((int64_t)t0 + 16 * u + v_tok, last_row);
            load_bytes<NB>(k_rows + krow * mrb, s.kw[u]);
            load_bytes<NB>(v_rows + vrow * mrb, s.vw[u]);
            if (AB) {
                s.kaux[u] = load_small<ABYTES>(ka_rows + krow * arb);
                s.vaux[u] = load_small<ABYTES>(va_rows + vrow * arb);
            }
            const int ts = t0 + 16 * u + 4 * grp;      // rows up to the plane capacity are readable
            s.ks[u] = *reinterpret_cast<const uint2 *>(ks_plane + ts);
            s.vs[u] = *reinterpret_cast<const uint2 *>(vs_plane + ts);
        }
    };

    FastTile<NW, AB> cur;
    if (t_begin < t_end) load_super(t_begin, cur);

    half4 qf[CPL];
    {
        const uint16_t *qp = (const uint16_t *)p.Q + b * p.qsb + hq * p.qsh + (int64_t)tq * p.qst + grp * CPL * 4;
#pragma unroll
        for (int j = 0; j < CPL; j++)
            qf[j] = col_ok ? chunk_to_half<DT>(*reinterpret_cast<const uint2 *>(qp + 4 * j)) : half4{0, 0, 0, 0};
    }

    fill_tables16<DT, NT>(ktab, (const uint2 *)p.Kc.joint + hkv * (p.Kc.jsh / 4), p.Kc.K,
                          vtab, (const uint2 *)p.Vc.joint + hkv * (p.Vc.jsh / 4), p.Vc.K);
    __syncthreads();

    // Scores are kept as v = S^T * rs (+ qmax * unscaled outlier part); the softmax argument is c_log2 * v.
    const float c = p.c_log2, qmaxf = (float)p.qmax;
    float m_run = -INFINITY, l_run = 0.f;
    float4v acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};

    for (int t0 = t_begin; t0 < t_end; t0 += kSuper) {
        FastTile<NW, AB> nxt;
        const bool more = t0 + kSuper < t_end;
        if (more) load_super(t0 + kSuper, nxt);

        float4v sT[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Kc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, col, grp * CPL, fl, sb_base);
            half4 a[CPL];
            decode_chunks<CPL, MB, AB, IB, NW>(cur.kw[u], AB ? cur.kaux[u] : 0u, ktab_b, idx_bits, a);
            float4v s = float4v{0.f, 0.f, 0.f, 0.f}, so = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                if (FLAGS) {
                    const bool f = (fl >> j) & 1u;
                    if (__builtin_amdgcn_ballot_w64(f) != 0) {
                        half4 ao = half4{0, 0, 0, 0};
                        if (f) {
                            ao = outlier_chunk(p.Kc, DT, bh, sb_base + __popc(fl & ((1u << j) - 1u)));
                            a[j] = half4{0, 0, 0, 0};
                        }
                        so = __builtin_amdgcn_mfma_f32_16x16x16f16(ao, qf[j], so, 0, 0, 0);
                    }
                }
                s = __builtin_amdgcn_mfma_f32_16x16x16f16(a[j], qf[j], s, 0, 0, 0);
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float rs = scale_f32<DT>(e < 2 ? cur.ks[u].x : cur.ks[u].y, e & 1);
                s[e] = s[e] * rs;
                if (FLAGS) s[e] = fmaf(so[e], qmaxf, s[e]);
            }
            sT[u] = s;
        }
        // ---- mask (boundary super-tiles only), online softmax ----
        if (!(t0 + kSuper <= lim_min && t0 + kSuper <= t_end)) {
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int t = t0 + 16 * u + 4 * grp + e;
                    if (!(t < col_lim && t < t_end)) sT[u][e] = -INFINITY;
                }
        }
        float tmax = fmaxf(fmaxf(fmaxf(sT[0][0], sT[0][1]), fmaxf(sT[0][2], sT[0][3])),
                           fmaxf(fmaxf(sT[1][0], sT[1][1]), fmaxf(sT[1][2], sT[1][3])));
        tmax = fmaxf(tmax, fmaxf(fmaxf(fmaxf(sT[2][0], sT[2][1]), fmaxf(sT[2][2], sT[2][3])),
                                 fmaxf(fmaxf(sT[3][0], sT[3][1]), fmaxf(sT[3][2], sT[3][3]))));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {     // rescale only when some column's maximum moved
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
            l_run *= alpha;
#pragma unroll
            for (int j = 0; j < CPL; j++) acc[j] = acc[j] * alpha;
            m_run = m_new;
        }
        const float mc = -m_use * c;
        half4 pT[4], pTo[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            float pe[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                pe[e] = __builtin_amdgcn_exp2f(fmaf(sT[u][e], c, mc));
                l_run += pe[e];
            }
            const half2v p01 = half2v{(_Float16)pe[0], (_Float16)pe[1]} * scale_h2<DT>(cur.vs[u].x);
            const half2v p23 = half2v{(_Float16)pe[2], (_Float16)pe[3]} * scale_h2<DT>(cur.vs[u].y);
            pT[u] = half4{p01[0], p01[1], p23[0], p23[1]};
            if (FLAGS) pTo[u] = half4{(_Float16)(pe[0] * qmaxf), (_Float16)(pe[1] * qmaxf), (_Float16)(pe[2] * qmaxf), (_Float16)(pe[3] * qmaxf)};
        }
        // ---- O^T += V^T . P^T (the 1/qmax of the radius is applied once, in the epilogue) ----
#pragma unroll
        for (int u = 0; u < 4; u++) {
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Vc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, v_tok, v_grp * CPL, fl, sb_base);
            half4 a[CPL];
            decode_chunks<CPL, MB, AB, IB, NW>(cur.vw[u], AB ? cur.vaux[u] : 0u, vtab_b, idx_bits, a);
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                if (FLAGS) {
                    const bool f = (fl >> j) & 1u;
                    if (__builtin_amdgcn_ballot_w64(f) != 0) {
                        half4 ao = half4{0, 0, 0, 0};
                        if (f) {
                            ao = outlier_chunk(p.Vc, DT, bh, sb_base + __popc(fl & ((1u << j) - 1u)));
                            a[j] = half4{0, 0, 0, 0};
                        }
                        uint2 ro = __builtin_bit_cast(uint2, ao);
                        quad_transpose(ro.x, ro.y, lane);
                        acc[j] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, ro), pTo[u], acc[j], 0, 0, 0);
                    }
                }
                uint2 r = __builtin_bit_cast(uint2, a[j]);
                quad_transpose(r.x, r.y, lane);
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, r), pT[u], acc[j], 0, 0, 0);
            }
        }
        if (more) cur = nxt;
    }

    // ---- merge the block's waves through LDS ----
    float l_tot = l_run;
    l_tot += __shfl_xor(l_tot, 16);
    l_tot += __shfl_xor(l_tot, 32);
    float *red = reinterpret_cast<float *>(lds_tab);            // [wave][16 cols][d_h + 2]
    __syncthreads();
    {
        float *wp = red + ((size_t)wave * 16 + col) * (d_h + 2);
        if (grp == 0) { wp[0] = m_run; wp[1] = l_tot; }
#pragma unroll
        for (int j = 0; j < CPL; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) wp[2 + grp * CPL * 4 + 4 * j + e] = acc[j][e];
    }
    __syncthreads();
    const int ncols = min(16, p.Tq * G - cg * 16);
    const float inv_qmax = p.inv_qmax;
    for (int o = threadIdx.x; o < ncols * d_h; o += NT) {
        const int cc = o / d_h, e = o - cc * d_h;
        const int ci = cg * 16 + cc;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < kFastWaves; w++) m = fmaxf(m, red[((size_t)w * 16 + cc) * (d_h + 2)]);
        float l = 0.f, a = 0.f;
        if (m > -INFINITY) {
#pragma unroll
            for (int w = 0; w < kFastWaves; w++) {
                const float *q = red + ((size_t)w * 16 + cc) * (d_h + 2);
                const float f = __builtin_amdgcn_exp2f((q[0] - m) * c);
                l = fmaf(q[1], f, l);
                a = fmaf(q[2 + e], f, a);
            }
        }
        const int tq2 = ci / G, hq2 = hkv * G + (ci - tq2 * G);
        if (p.n_splits == 1) {
            store_any(p.O, DT, b * p.osb + hq2 * p.osh + (int64_t)tq2 * p.ost + e, l > 0.f ? a * inv_qmax / l : 0.f);
        } else {
            // partials carry the maximum in softmax units (base-2 exponent) and acc already divided by qmax
            float *wp = p.ws + ((((size_t)b * p.Hq + hq2) * p.Tq + tq2) * p.n_splits + sp) * (size_t)(d_h + 2);
            if (e == 0) { wp[0] = m * c; wp[1] = l; }
            wp[2 + e] = a * inv_qmax;
        }
    }
}

template <int CPL, int MB, int AB, int IB, int DT>
static int launch_one(const AttnParams &p, bool flags, dim3 grid, size_t table_bytes, hipStream_t st) {
    // LDS: K table at 0, V table at kVTabOffset; reused afterwards for the cross-wave merge [wave][16][d_h + 2] floats
    (void)table_bytes;
    size_t shmem = (size_t)kVTabOffset + (size_t)p.Vc.K * 8;
    const size_t merge = (size_t)kFastWaves * 16 * (16 * CPL + 2) * sizeof(float);
    if (shmem < merge) shmem = merge;
    auto kern = flags ? attn_fast_kernel<CPL, MB, AB, IB, DT, true> : attn_fast_kernel<CPL, MB, AB, IB, DT, false>;
    if (shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(kern, grid, dim3(kFastWaves * 64), shmem, st, p);
    return hip_status(hipGetLastError());
}

template <int CPL, int DT>
static int launch_layout(const AttnParams &p, int mb, bool flags, dim3 grid, size_t table_bytes, hipStream_t st, bool *handled) {
    if (p.Kc.K > kVTabOffset / 8 || p.Vc.K > kVTabOffset / 8) return HQMQ_OK;     // tables beyond the fixed LDS slots
    *handled = true;
    if (mb == 16 && p.aux_bits == 0 && p.idx_bits == 12) return launch_one<CPL, 16, 0, 12, DT>(p, flags, grid, table_bytes, st);
    if (mb == 16 && p.aux_bits == 0) return launch_one<CPL, 16, 0, 0, DT>(p, flags, grid, table_bytes, st);
    if (mb == 12 && p.aux_bits == 1 && CPL == 8) return launch_one<8, 12, 1, 0, DT>(p, flags, grid, table_bytes, st);
    if (mb == 16 && p.aux_bits == 3 && CPL == 8) return launch_one<8, 16, 3, 0, DT>(p, flags, grid, table_bytes, st);
    *handled = false;
    return HQMQ_OK;
}

int launch_attn_fast(const AttnParams &p, int main_bits, bool flags, dim3 grid, size_t table_bytes, hipStream_t st, bool *handled) {
    *handled = false;
    if (p.dtype != HQMQ_F16 && p.dtype != HQMQ_BF16) return HQMQ_OK;
    if (p.n != 16 && p.n != 32) return HQMQ_OK;
    // 8-byte vector loads of Q rows, table rows and sideband chunks; strides were checked by the caller
    if (p.n == 32) {
        if (p.dtype == HQMQ_F16) return launch_layout<8, HQMQ_F16>(p, main_bits, flags, grid, table_bytes, st, handled);
        return launch_layout<8, HQMQ_BF16>(p, main_bits, flags, grid, table_bytes, st, handled);
    }
    if (p.dtype == HQMQ_F16) return launch_layout<4, HQMQ_F16>(p, main_bits, flags, grid, table_bytes, st, handled);
    return launch_layout<4, HQMQ_BF16>(p, main_bits, flags, grid, table_bytes, st, handled);
}

}  // namespace hqmq
