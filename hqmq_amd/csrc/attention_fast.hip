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

template <int DT>
__device__ __forceinline__ void fill_table16(uint2 *dst, const uint2 *src, int K) {
    constexpr int U = 6;
    for (int k0 = threadIdx.x; k0 < K; k0 += 256 * U) {
        uint2 tmp[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * 256;
            tmp[u] = k < K ? src[k] : uint2{0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * 256;
            if (k < K) dst[k] = __builtin_bit_cast(uint2, chunk_to_half<DT>(tmp[u]));
        }
    }
}

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

template <int CPL, int MB, int AB, int DT, bool FLAGS>
__global__ __launch_bounds__(kAttnWaves * 64, 2) void attn_fast_kernel(AttnParams p) {
    constexpr int NB = CPL * MB / 8;
    constexpr int NW = (NB + 3) / 4;
    constexpr int ABYTES = CPL * AB / 8;     // aux bytes per lane (CPL * AB is a multiple of 8 here)
    static_assert(AB == 0 || (CPL * AB) % 8 == 0, "aux bits of one lane must be whole bytes");
    extern __shared__ uint2 lds_tab[];
    uint2 *ktab = lds_tab, *vtab = lds_tab + p.Kc.K;

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
    int blk_lim = col_lim;
    for (int o = 1; o < 16; o <<= 1) blk_lim = max(blk_lim, __shfl_xor(blk_lim, o));
    int per_split = (blk_lim + p.n_splits - 1) / p.n_splits;
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int b_begin = min(sp * per_split, blk_lim), b_end = min(blk_lim, b_begin + per_split);
    int per_wave = (b_end - b_begin + kAttnWaves - 1) / kAttnWaves;
    per_wave = (per_wave + kSuper - 1) / kSuper * kSuper;
    const int t_begin = min(b_begin + wave * per_wave, b_end), t_end = min(b_end, t_begin + per_wave);

    const size_t plane_row0 = (size_t)bh * p.t_cap;
    constexpr int mrb = n * MB / 8, arb = (n * AB + 7) / 8, frb = (n + 7) / 8;
    const int64_t tiles_cap = (p.t_cap + kTile - 1) / kTile;
    const uint32_t idx_mask = (1u << p.idx_bits) - 1u;
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

    fill_table16<DT>(ktab, (const uint2 *)p.Kc.joint + hkv * (p.Kc.jsh / 4), p.Kc.K);
    fill_table16<DT>(vtab, (const uint2 *)p.Vc.joint + hkv * (p.Vc.jsh / 4), p.Vc.K);
    __syncthreads();

    float m_run = -INFINITY, l_run = 0.f;
    float4v acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};

    auto decode = [&](const uint32_t (&w)[NW], uint32_t aux, int j, const uint2 *tab) -> half4 {
        uint32_t code = code_at<MB, NW>(w, j);
        if (AB) code |= ((aux >> (j * AB)) & ((1u << AB) - 1u)) << MB;
        const _Float16 rq = (_Float16)(uint16_t)(code >> idx_bits);
        half4 a = __builtin_bit_cast(half4, tab[code & idx_mask]);
        return a * rq;
    };

    for (int t0 = t_begin; t0 < t_end; t0 += kSuper) {
        FastTile<NW, AB> nxt;
        const bool more = t0 + kSuper < t_end;
        if (more) load_super(t0 + kSuper, nxt);

        float4v sT[4], sTo[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Kc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, col, grp * CPL, fl, sb_base);
            half4 a[CPL];
#pragma unroll
            for (int j = 0; j < CPL; j++) a[j] = decode(cur.kw[u], AB ? cur.kaux[u] : 0u, j, ktab);
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
            sT[u] = s;
            if (FLAGS) sTo[u] = so;
        }
        // ---- scale, mask, online softmax ----
        float tmax = -INFINITY;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t raw[2] = {cur.ks[u].x, cur.ks[u].y};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int t = t0 + 16 * u + 4 * grp + e;
                const float rs = cvt16<DT>((raw[e >> 1] >> (16 * (e & 1))) & 0xffffu);
                float v = sT[u][e] * (rs * p.c_log2);
                if (FLAGS) v = fmaf(sTo[u][e], p.c_plain, v);
                v = (t < col_lim && t < t_end) ? v : -INFINITY;
                sT[u][e] = v;
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
            const uint32_t raw[2] = {cur.vs[u].x, cur.vs[u].y};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float pe = exp2f(sT[u][e] - m_use);
                l_run += pe;
                const float rs = cvt16<DT>((raw[e >> 1] >> (16 * (e & 1))) & 0xffffu);
                pT[u][e] = (_Float16)(pe * (rs * p.inv_qmax));
                if (FLAGS) pTo[u][e] = (_Float16)pe;
            }
        }
        // ---- O^T += V^T . P^T ----
#pragma unroll
        for (int u = 0; u < 4; u++) {
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Vc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, v_tok, v_grp * CPL, fl, sb_base);
            half4 a[CPL];
#pragma unroll
            for (int j = 0; j < CPL; j++) a[j] = decode(cur.vw[u], AB ? cur.vaux[u] : 0u, j, vtab);
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

    // ---- merge the block's waves through LDS, then write the output or this block's partial ----
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
    for (int o = threadIdx.x; o < 16 * d_h; o += kAttnWaves * 64) {
        const int c = o / d_h, e = o - c * d_h;
        const int ci = cg * 16 + c;
        if (ci >= p.Tq * G) continue;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) m = fmaxf(m, red[((size_t)w * 16 + c) * (d_h + 2)]);
        float l = 0.f, a = 0.f;
        if (m > -INFINITY) {
#pragma unroll
            for (int w = 0; w < kAttnWaves; w++) {
                const float *q = red + ((size_t)w * 16 + c) * (d_h + 2);
                const float f = exp2f(q[0] - m);
                l = fmaf(q[1], f, l);
                a = fmaf(q[2 + e], f, a);
            }
        }
        const int tq2 = ci / G, hq2 = hkv * G + (ci - tq2 * G);
        if (p.n_splits == 1) {
            store_any(p.O, DT, b * p.osb + hq2 * p.osh + (int64_t)tq2 * p.ost + e, l > 0.f ? a / l : 0.f);
        } else {
            float *wp = p.ws + ((((size_t)b * p.Hq + hq2) * p.Tq + tq2) * p.n_splits + sp) * (size_t)(d_h + 2);
            if (e == 0) { wp[0] = m; wp[1] = l; }
            wp[2 + e] = a;
        }
    }
}

template <int CPL, int MB, int AB, int DT>
static int launch_one(const AttnParams &p, bool flags, dim3 grid, size_t shmem, hipStream_t st) {
    auto kern = flags ? attn_fast_kernel<CPL, MB, AB, DT, true> : attn_fast_kernel<CPL, MB, AB, DT, false>;
    if (shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(kern, grid, dim3(kAttnWaves * 64), shmem, st, p);
    return hip_status(hipGetLastError());
}

template <int CPL, int DT>
static int launch_layout(const AttnParams &p, int mb, bool flags, dim3 grid, size_t shmem, hipStream_t st, bool *handled) {
    *handled = true;
    if (mb == 16 && p.aux_bits == 0) return launch_one<CPL, 16, 0, DT>(p, flags, grid, shmem, st);
    if (mb == 12 && p.aux_bits == 1 && CPL == 8) return launch_one<8, 12, 1, DT>(p, flags, grid, shmem, st);
    if (mb == 16 && p.aux_bits == 3 && CPL == 8) return launch_one<8, 16, 3, DT>(p, flags, grid, shmem, st);
    *handled = false;
    return HQMQ_OK;
}

int launch_attn_fast(const AttnParams &p, int main_bits, bool flags, dim3 grid, size_t shmem, hipStream_t st, bool *handled) {
    *handled = false;
    if (p.dtype != HQMQ_F16 && p.dtype != HQMQ_BF16) return HQMQ_OK;
    if (p.n != 16 && p.n != 32) return HQMQ_OK;
    // 8-byte vector loads of Q rows, table rows and sideband chunks; strides were checked by the caller
    if (p.n == 32) {
        if (p.dtype == HQMQ_F16) return launch_layout<8, HQMQ_F16>(p, main_bits, flags, grid, shmem, st, handled);
        return launch_layout<8, HQMQ_BF16>(p, main_bits, flags, grid, shmem, st, handled);
    }
    if (p.dtype == HQMQ_F16) return launch_layout<4, HQMQ_F16>(p, main_bits, flags, grid, shmem, st, handled);
    return launch_layout<4, HQMQ_BF16>(p, main_bits, flags, grid, shmem, st, handled);
}

}  // namespace hqmq
