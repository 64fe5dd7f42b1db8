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
#include "attention_common.h"
#include <mutex>

namespace hqmq {

// Raw codes, aux bits and per-token scales of one 64-token super-tile, as one lane needs them:
// K side (token = lane % 16 of each tile, code group = lane / 16) and V side (token = 4*(lane/16) + lane%4,
// code group = (lane % 16) / 4); scales of the 4 tokens 4*(lane/16) + 0..3 of each tile (S^T / P^T rows).
template <int NW>
struct SuperTile {
    uint32_t kw[4][NW], vw[4][NW];
    uint64_t kaux[4], vaux[4];
    float ks[4][4], vs[4][4];
};

__device__ __forceinline__ void load_scales4(const void *plane, int dtype, int64_t base, int64_t st, bool vec, int t, int Tkv,
                                             float (&out)[4]) {
    if (vec) {  // 4 consecutive tokens, t % 4 == 0, rows up to the plane capacity are readable
        if (dtype == HQMQ_F32) {
            const float4 v = *reinterpret_cast<const float4 *>((const float *)plane + base + t);
            out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
        } else {
            const uint2 v = *reinterpret_cast<const uint2 *>((const uint16_t *)plane + base + t);
            if (dtype == HQMQ_F16) {
                const half4 h = __builtin_bit_cast(half4, v);
                out[0] = (float)h[0]; out[1] = (float)h[1]; out[2] = (float)h[2]; out[3] = (float)h[3];
            } else {
                out[0] = __uint_as_float(v.x << 16); out[1] = __uint_as_float(v.x & 0xffff0000u);
                out[2] = __uint_as_float(v.y << 16); out[3] = __uint_as_float(v.y & 0xffff0000u);
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) out[e] = (t + e < Tkv) ? load_any(plane, dtype, base + (int64_t)(t + e) * st) : 0.f;
    }
}

template <int CPL, int MB, bool FLAGS>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_kernel(AttnParams p) {
    constexpr int NB = CPL * MB / 8;
    constexpr int NW = (NB + 3) / 4;
    extern __shared__ uint2 lds_tab[];
    uint2 *ktab = lds_tab, *vtab = lds_tab + p.Kc.K;

    // blocks are dispatched in grid order: batch_order lists the sequences in the order they should start
    // (longest first for ragged batches, so that no long sequence is left for the end)
    const int slot = blockIdx.z / p.Hkv, hkv = blockIdx.z - slot * p.Hkv;
    const int b = p.batch_order ? min(max(p.batch_order[slot], 0), p.B - 1) : slot;
    const int bh = b * p.Hkv + hkv;
    const int cg = blockIdx.y, sp = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int dtype = p.dtype;
    const int n = p.n, G = p.G;
    const int col = lane & 15, grp = lane >> 4;
    const int cidx = cg * 16 + col;
    const bool col_ok = cidx < p.Tq * G;
    const int tq = col_ok ? cidx / G : 0, g = col_ok ? cidx - tq * G : 0;
    const int hq = hkv * G + g;

    // ---- KV range of this block and of this wave ----
    int kv_end = p.kv_len ? p.kv_len[b] : p.Tkv;
    kv_end = min(max(kv_end, 0), p.Tkv);
    int64_t lim64 = kv_end;                       // per-column visible limit (exclusive)
    if (p.causal) lim64 = min(lim64, (int64_t)tq + p.causal_offset + 1);
    if (!col_ok || lim64 < 0) lim64 = 0;
    const int col_lim = (int)lim64;
    int blk_lim = col_lim;                        // block-wide limit: max over the 16 columns
    for (int o = 1; o < 16; o <<= 1) blk_lim = max(blk_lim, __shfl_xor(blk_lim, o));
    // tokens before kv_start[b] are invisible (left padding): the walk starts at the super-tile that holds it
    const int col_start = p.kv_start ? min(max(p.kv_start[b], 0), blk_lim) : 0;
    const int blk_lo = col_start / kSuper * kSuper;
    int per_split = (blk_lim - blk_lo + p.n_splits - 1) / p.n_splits;
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int b_begin = min(blk_lo + sp * per_split, blk_lim), b_end = min(blk_lim, b_begin + per_split);
    int per_wave = (b_end - b_begin + kAttnWaves - 1) / kAttnWaves;
    per_wave = (per_wave + kSuper - 1) / kSuper * kSuper;
    const int t_begin = min(b_begin + wave * per_wave, b_end), t_end = min(b_end, t_begin + per_wave);

    const size_t plane_row0 = (size_t)bh * p.t_cap;
    const int mrb = n * MB / 8;
    const int arb = (n * p.aux_bits + 7) >> 3;
    const int frb = (n + 7) >> 3;
    const int64_t tiles_cap = (p.t_cap + kTile - 1) / kTile;
    const uint32_t idx_mask = (1u << p.idx_bits) - 1u;
    const int idx_bits = p.idx_bits, ab = p.aux_bits;
    const int v_tok = 4 * grp + (col & 3), v_grp = col >> 2;   // V-side lane role
    const int64_t ks_base = b * p.Kc.ssb + hkv * p.Kc.ssh, vs_base = b * p.Vc.ssb + hkv * p.Vc.ssh;

    auto load_super = [&](int t0, SuperTile<NW> &s) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int64_t krow = min((int64_t)t0 + 16 * u + col, p.t_cap - 1);
            const int64_t vrow = min((int64_t)t0 + 16 * u + v_tok, p.t_cap - 1);
            load_bytes<NB>(p.Kc.main_plane + (plane_row0 + krow) * mrb + grp * NB, s.kw[u]);
            load_bytes<NB>(p.Vc.main_plane + (plane_row0 + vrow) * mrb + v_grp * NB, s.vw[u]);
            s.kaux[u] = s.vaux[u] = 0;
            if (ab) {
                s.kaux[u] = load_aux<CPL>(p.Kc.aux_plane + (plane_row0 + krow) * arb, arb, grp * CPL, ab);
                s.vaux[u] = load_aux<CPL>(p.Vc.aux_plane + (plane_row0 + vrow) * arb, arb, v_grp * CPL, ab);
            }
            const int ts = t0 + 16 * u + 4 * grp;
            load_scales4(p.Kc.scale_plane, dtype, ks_base, p.Kc.sst, p.scale_vec, ts, p.Tkv, s.ks[u]);
            load_scales4(p.Vc.scale_plane, dtype, vs_base, p.Vc.sst, p.scale_vec, ts, p.Tkv, s.vs[u]);
        }
    };

    // the first super-tile's loads fly while the codeword tables are copied to LDS
    SuperTile<NW> cur;
    if (t_begin < t_end) load_super(t_begin, cur);

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

    // ---- per-head codeword tables -> LDS as fp16 ----
    fill_table(ktab, p.Kc.joint, dtype, hkv * (p.Kc.jsh / 4), p.Kc.K);
    fill_table(vtab, p.Vc.joint, dtype, hkv * (p.Vc.jsh / 4), p.Vc.K);
    __syncthreads();

    float m_run = -INFINITY, l_run = 0.f;
    float4v acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};
    // Range guard of bf16 / fp32 caches (see attention_common.h): the softmax weights carry 2^-eshift, so that
    // P * (V scale) fits fp16; verbatim outlier chunks are brought into range by the same bounds (a verbatim value
    // never exceeds its token's scale) and meet the weights without the offset (V) or are rescaled in fp32 (K).
    const float eshift = v_scale_shift(p.Vc), kshift = FLAGS ? v_scale_shift(p.Kc) : 0.f;
    const float v_down = exp2f(-eshift), p_up = exp2f(eshift), k_down = exp2f(-kshift), k_up = exp2f(kshift) * p.c_plain;

    for (int t0 = t_begin; t0 < t_end; t0 += kSuper) {
        SuperTile<NW> nxt;
        const bool more = t0 + kSuper < t_end;
        if (more) load_super(t0 + kSuper, nxt);

        float4v sT[4], sTo[4];
        // ---------------- S^T = K . Q^T for 4 tiles ----------------
#pragma unroll
        for (int u = 0; u < 4; u++) {
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Kc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, col, grp * CPL, fl, sb_base);
            float4v s = float4v{0.f, 0.f, 0.f, 0.f}, so = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                uint32_t code = code_at<MB, NW>(cur.kw[u], j);
                if (ab) code |= (uint32_t)((cur.kaux[u] >> (j * ab)) & ((1u << ab) - 1u)) << MB;
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
                            ao = outlier_chunk(p.Kc, dtype, bh, sb_base + __popc(fl & ((1u << j) - 1u)), k_down);
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
                float v = sT[u][e] * (cur.ks[u][e] * p.c_log2);
                if (FLAGS) v = fmaf(sTo[u][e], k_up, v);
                v = (t < col_lim && t < t_end && t >= col_start) ? v : -INFINITY;
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
                const float pe = exp2f(pv[u][e] - m_use - eshift);
                l_run += pe;
                pT[u][e] = (_Float16)(pe * (cur.vs[u][e] * p.inv_qmax));
                if (FLAGS) pTo[u][e] = (_Float16)(pe * p_up);          // without the offset: at most 1
            }
        }
        // ---------------- O^T += V^T . P^T ----------------
#pragma unroll
        for (int u = 0; u < 4; u++) {
            uint32_t fl = 0;
            int sb_base = 0;
            if (FLAGS)
                tile_flags<CPL>(p.Vc, plane_row0, (int64_t)t0 + 16 * u, p.t_cap, frb,
                                (size_t)bh * tiles_cap + min((int64_t)((t0 + 16 * u) >> 4), tiles_cap - 1), col, v_tok, v_grp * CPL, fl, sb_base);
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                uint32_t code = code_at<MB, NW>(cur.vw[u], j);
                if (ab) code |= (uint32_t)((cur.vaux[u] >> (j * ab)) & ((1u << ab) - 1u)) << MB;
                const uint32_t k = code & idx_mask;
                const _Float16 rq = (_Float16)(float)(code >> idx_bits);
                half4 a = __builtin_bit_cast(half4, vtab[k]);
                a = a * rq;
                if (FLAGS) {
                    const bool f = (fl >> j) & 1u;
                    if (__builtin_amdgcn_ballot_w64(f) != 0) {
                        half4 ao = half4{0, 0, 0, 0};
                        if (f) {
                            ao = outlier_chunk(p.Vc, dtype, bh, sb_base + __popc(fl & ((1u << j) - 1u)), v_down);
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
        if (more) cur = nxt;
    }

    // ---- merge the block's waves through LDS (the tables are no longer needed) ----
    // lane (col, grp) holds, for block j, dims 4*(CPL*grp + j) + 0..3 of column col
    float l_tot = l_run;
    l_tot += __shfl_xor(l_tot, 16);
    l_tot += __shfl_xor(l_tot, 32);
    const int d_h = 4 * n;
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
    for (int o = threadIdx.x; o < 16 * d_h; o += blockDim.x) {
        const int c = o / d_h, e = o - c * d_h;
        const int ci = cg * 16 + c;
        if (ci >= p.Tq * G) continue;
        float m = -INFINITY;
        for (int w = 0; w < kAttnWaves; w++) m = fmaxf(m, red[((size_t)w * 16 + c) * (d_h + 2)]);
        float l = 0.f, a = 0.f;
        if (m > -INFINITY) {
            for (int w = 0; w < kAttnWaves; w++) {
                const float *q = red + ((size_t)w * 16 + c) * (d_h + 2);
                const float f = exp2f(q[0] - m);
                l = fmaf(q[1], f, l);
                a = fmaf(q[2 + e], f, a);
            }
        }
        const int tq2 = ci / G, hq2 = hkv * G + (ci - tq2 * G);
        if (p.n_splits == 1) {
            store_any(p.O, dtype, b * p.osb + hq2 * p.osh + (int64_t)tq2 * p.ost + e, l > 0.f ? a / l : 0.f);
        } else {
            float *wp = p.ws + ((((size_t)b * p.Hq + hq2) * p.Tq + tq2) * p.n_splits + sp) * (size_t)(d_h + kPartialHead);
            if (e == 0) { wp[0] = m; wp[1] = l; }
            wp[kPartialHead + e] = a;
        }
    }
}

// Merge of the split partials: one block of 256 threads per output row.  A thread owns four consecutive output
// elements (one 16-byte load per split) and every (256 / (d_h / 4))-th split; it loads its splits in batches of four
// independent (m, l) and acc loads, merges them in registers, and the split groups merge through LDS.  At 32 splits
// and d_h 128 that is one batch of eight loads per thread: the kernel costs one round trip to memory, one barrier
// and the launch.
constexpr int kCombineThreads = 256;
__global__ __launch_bounds__(kCombineThreads) void attn_combine_kernel(const float *ws, void *O, int dtype, int Hq, int Tq, int d_h,
                                                                       int n_splits, int64_t osb, int64_t osh, int64_t ost) {
    __shared__ float red[kCombineThreads * 6];
    const unsigned row = blockIdx.x;
    const int ncol = d_h >> 2, groups = kCombineThreads / ncol;           // d_h <= 256: at least four groups
    const int c4 = threadIdx.x % ncol, grp = threadIdx.x / ncol;
    const int rec = d_h + kPartialHead;
    const float *base = ws + (size_t)row * (size_t)n_splits * rec;
    float M = -INFINITY, L = 0.f;
    float4v A = float4v{0.f, 0.f, 0.f, 0.f};
    if (grp < groups) {
        constexpr int SC = 4;
        for (int s0 = grp; s0 < n_splits; s0 += SC * groups) {
            float2 ml[SC];
            float4v as[SC];
#pragma unroll
            for (int i = 0; i < SC; i++) {
                const int s = s0 + i * groups;
                const float *q = base + (size_t)min(s, n_splits - 1) * rec;
                ml[i] = *reinterpret_cast<const float2 *>(q);
                as[i] = *reinterpret_cast<const float4v *>(q + kPartialHead + 4 * c4);
                if (s >= n_splits) { ml[i] = float2{-INFINITY, 0.f}; as[i] = float4v{0.f, 0.f, 0.f, 0.f}; }
            }
            float mx = M;
#pragma unroll
            for (int i = 0; i < SC; i++) mx = fmaxf(mx, ml[i].x);
            if (mx > -INFINITY) {
                const float f = __builtin_amdgcn_exp2f(M - mx);          // 0 while M is still -inf
                L *= f;
                A = A * f;
#pragma unroll
                for (int i = 0; i < SC; i++) {
                    const float w = __builtin_amdgcn_exp2f(ml[i].x - mx);
                    L = fmaf(ml[i].y, w, L);
                    A = A + as[i] * w;
                }
                M = mx;
            }
        }
        float *r = red + (size_t)threadIdx.x * 6;
        r[0] = M; r[1] = L; r[2] = A[0]; r[3] = A[1]; r[4] = A[2]; r[5] = A[3];
    }
    __syncthreads();
    if (grp != 0) return;
    // the groups' results: the maximum first (independent reads), then one weight per group, in batches of eight
    float mx = M;
    for (int g = 1; g < groups; g++) mx = fmaxf(mx, red[(size_t)(g * ncol + c4) * 6]);
    if (mx > -INFINITY) {
        const float f = __builtin_amdgcn_exp2f(M - mx);
        L *= f;
        A = A * f;
        for (int g0 = 1; g0 < groups; g0 += 8) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int g = g0 + i;
                if (g < groups) {
                    const float *r = red + (size_t)(g * ncol + c4) * 6;
                    const float w = __builtin_amdgcn_exp2f(r[0] - mx);      // -inf - finite = -inf -> 0
                    L = fmaf(r[1], w, L);
                    A = A + float4v{r[2], r[3], r[4], r[5]} * w;
                }
            }
        }
    }
    const unsigned bh = row / (unsigned)Tq, tq = row - bh * (unsigned)Tq, b = bh / (unsigned)Hq, hq = bh - b * (unsigned)Hq;
    const int64_t o = (int64_t)b * osb + (int64_t)hq * osh + (int64_t)tq * ost + 4 * c4;
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = L > 0.f ? A[e] / L : 0.f;
    if (dtype != HQMQ_F32 && ((((uintptr_t)O) | (uintptr_t)(osb * 2) | (uintptr_t)(osh * 2) | (uintptr_t)(ost * 2)) & 7) == 0) {
        // four 16-bit results as one 8-byte store
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++) h[e] = dtype == HQMQ_F16 ? __half_as_ushort(__float2half_rn(r[e])) : f32_to_bf16_bits(r[e]);
        *reinterpret_cast<uint2 *>((uint16_t *)O + o) = uint2{(uint32_t)h[0] | (uint32_t)h[1] << 16, (uint32_t)h[2] | (uint32_t)h[3] << 16};
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) store_any(O, dtype, o + e, r[e]);
    }
}

// op over all 64 lanes, the result in every lane: quad and row permutations (DPP), then the 16- and 32-lane swaps
template <class Op>
__device__ __forceinline__ float wave_reduce(float x, Op op) {
    auto dpp = [](float v, int ctrl_quad) {
        const int b = __builtin_bit_cast(int, v);
        int r;
        switch (ctrl_quad) {
            case 0: r = __builtin_amdgcn_update_dpp(0, b, 0xB1, 0xF, 0xF, false); break;     // quad_perm [1,0,3,2]
            case 1: r = __builtin_amdgcn_update_dpp(0, b, 0x4E, 0xF, 0xF, false); break;     // quad_perm [2,3,0,1]
            case 2: r = __builtin_amdgcn_update_dpp(0, b, 0x141, 0xF, 0xF, false); break;    // row_half_mirror
            default: r = __builtin_amdgcn_update_dpp(0, b, 0x140, 0xF, 0xF, false); break;   // row_mirror
        }
        return __builtin_bit_cast(float, r);
    };
    x = op(x, dpp(x, 0));
    x = op(x, dpp(x, 1));
    x = op(x, dpp(x, 2));
    x = op(x, dpp(x, 3));
    const uint32_t b = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    x = op(__uint_as_float(r[0]), __uint_as_float(r[1]));
    const uint32_t c = __float_as_uint(x);
    const auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
    return op(__uint_as_float(q[0]), __uint_as_float(q[1]));
}

// The same merge for the common decode shape (d_h = 128, at most 32 splits, 16-bit output): one wavefront per row and
// no LDS.  A lane owns two output elements and loads them from all 32 split records at once (8 bytes each, 512 bytes
// per wavefront and record), together with the (m, l) pair of split (lane & 31): one round trip to memory.  The
// maximum and the denominator are reduced across the lanes, the 32 weights are read back lane by lane into scalar
// registers and multiply the records in place.
__global__ __launch_bounds__(64) void attn_combine_wave_kernel(const float *__restrict__ ws, uint16_t *__restrict__ O, int dtype, int Hq, int Tq,
                                                              int n_splits, int64_t osb, int64_t osh, int64_t ost) {
    constexpr int d_h = 128, rec = d_h + kPartialHead, NS = 32;
    const unsigned row = blockIdx.x;
    const int lane = threadIdx.x;
    const float *base = ws + (size_t)row * (size_t)n_splits * rec;
    const int sl = lane & 31;
    float2 ml = *reinterpret_cast<const float2 *>(base + (size_t)min(sl, n_splits - 1) * rec);
    float2 as[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) as[s] = *reinterpret_cast<const float2 *>(base + (size_t)min(s, n_splits - 1) * rec + kPartialHead + 2 * lane);
    if (sl >= n_splits) ml = float2{-INFINITY, 0.f};
    // reductions over the wavefront inside the vector unit (lane permutations, no LDS round trips): the upper half
    // repeats the lower one, so it takes no part in the sum
    const float M = wave_reduce(ml.x, [](float p, float q) { return fmaxf(p, q); });
    const float w = M > -INFINITY ? __builtin_amdgcn_exp2f(ml.x - M) : 0.f;        // -inf - finite = -inf -> 0
    const float L = wave_reduce(lane < 32 ? ml.y * w : 0.f, [](float p, float q) { return p + q; });
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const float wsc = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, w), s));
        a0 = fmaf(as[s].x, wsc, a0);
        a1 = fmaf(as[s].y, wsc, a1);
    }
    const float r0 = L > 0.f ? a0 / L : 0.f, r1 = L > 0.f ? a1 / L : 0.f;
    const unsigned bh = row / (unsigned)Tq, tq = row - bh * (unsigned)Tq, b = bh / (unsigned)Hq, hq = bh - b * (unsigned)Hq;
    const int64_t o = (int64_t)b * osb + (int64_t)hq * osh + (int64_t)tq * ost + 2 * lane;
    const uint32_t h0 = dtype == HQMQ_F16 ? __half_as_ushort(__float2half_rn(r0)) : f32_to_bf16_bits(r0);
    const uint32_t h1 = dtype == HQMQ_F16 ? __half_as_ushort(__float2half_rn(r1)) : f32_to_bf16_bits(r1);
    *reinterpret_cast<uint32_t *>(O + o) = h0 | h1 << 16;
}

static PackedDev to_dev(const hqmq_packed &k) {
    return PackedDev{k.main_plane, k.aux_plane, k.flag_plane, k.scale_plane, k.scale_sb, k.scale_sh, k.scale_st,
                     k.sideband, k.sb_tile_off, k.sb_cap, k.sb_coord, k.sb_count, k.joint, k.joint_sh, k.K, k.scale_max_bits};
}

template <int CPL, int MB>
static int launch_attn(const AttnParams &p, bool flags, dim3 grid, size_t shmem, hipStream_t st, const LaunchTiming &tm) {
    auto kern = flags ? attn_kernel<CPL, MB, true> : attn_kernel<CPL, MB, false>;
    if (shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    launch_timed(kern, grid, dim3(kAttnWaves * 64), shmem, st, tm, p);
    return hip_status(hipGetLastError());
}

template <int CPL>
static int launch_attn_mb(const AttnParams &p, int mb, bool flags, dim3 grid, size_t shmem, hipStream_t st, const LaunchTiming &tm) {
    switch (mb) {
        case 8: return launch_attn<CPL, 8>(p, flags, grid, shmem, st, tm);
        case 12:
            if constexpr (CPL % 2 == 0) return launch_attn<CPL, 12>(p, flags, grid, shmem, st, tm);
            else return HQMQ_ERR_SHAPE;
        case 16: return launch_attn<CPL, 16>(p, flags, grid, shmem, st, tm);
        default: return HQMQ_ERR_LAYOUT;
    }
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int64_t hqmq_attn_workspace_bytes(int B, int H_q, int T_q, int d_h, int n_splits) {
    if (n_splits <= 1) return 0;
    return (int64_t)B * H_q * T_q * n_splits * (d_h + kPartialHead) * 4;
}

// Blocks per (sequence, KV head, column group): one block per CU, blocks of at least 128 tokens (short contexts are
// bound by the launch's fixed costs: more, shorter blocks are faster down to that size even though half of such a
// block's wavefronts have no half-step).
extern "C" int hqmq_attn_pick_splits(int B, int H_q, int H_kv, int T_q, int T_kv, int ragged) {
    if (B < 1 || H_q < 1 || H_kv < 1 || T_q < 1 || T_kv < 1) return 1;
    const int G = H_q / H_kv;
    const int64_t base = (int64_t)B * H_kv * ((T_q * G + 15) / 16);
    // sequences of different lengths: two rounds of blocks, started longest first (batch_order), even out the finishing
    // times (config 4, 512 (sequence, head) pairs: 248 us with one block per pair, 264 with two, 287 with four)
    const int64_t target = ragged ? 512 : 256;
    int64_t s = (target + base - 1) / base;
    const int64_t cap = (T_kv + 2 * kSuper - 1) / (2 * kSuper);       // blocks of at least 128 tokens (4k tokens: 32 splits, 8.7 against 8.95 us)
    if (s > cap) s = cap;
    if (s < 1) s = 1;
    if (s > 512) s = 512;
    return (int)s;
}

extern "C" int hqmq_attn_combine(const void *workspace, void *O, int dtype, int B, int H_q, int T_q, int d_h, int n_splits,
                                 int64_t o_sb, int64_t o_sh, int64_t o_st, void *stream) {
    if (!workspace || !O) return HQMQ_ERR_NULL;
    if (B < 1 || H_q < 1 || T_q < 1 || d_h < 4 || d_h > 256 || (d_h & 3) || n_splits < 1 || n_splits > 8192) return HQMQ_ERR_SHAPE;
    if (dtype != HQMQ_F32 && dtype != HQMQ_F16 && dtype != HQMQ_BF16) return HQMQ_ERR_DTYPE;
    const int64_t rows = (int64_t)B * H_q * T_q;
    if (rows > 0x7fffffff) return HQMQ_ERR_SHAPE;
    if ((uintptr_t)workspace & 15) return HQMQ_ERR_ALIGN;
    if (d_h == 128 && n_splits <= 32 && dtype != HQMQ_F32 && ((((uintptr_t)O) | (uintptr_t)(o_sb * 2) | (uintptr_t)(o_sh * 2) | (uintptr_t)(o_st * 2)) & 3) == 0) {
        hipLaunchKernelGGL(attn_combine_wave_kernel, dim3((unsigned)rows), dim3(64), 0, (hipStream_t)stream, (const float *)workspace,
                           (uint16_t *)O, dtype, H_q, T_q, n_splits, o_sb, o_sh, o_st);
        return hip_status(hipGetLastError());
    }
    hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)rows), dim3(kCombineThreads), 0, (hipStream_t)stream,
                       (const float *)workspace, O, dtype, H_q, T_q, d_h, n_splits, o_sb, o_sh, o_st);
    return hip_status(hipGetLastError());
}

static int attn_fwd_impl(const hqmq_attn_args *a, void *stream) {
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
    // d_h in {16, 32, 64, 128, 256} and, for heads padded from sizes such as 80 or 160, {80, 160}
    if (n < 4 || n > 64 || (n & 3) || a->qmax < 1) return HQMQ_ERR_SHAPE;
    if ((n & (n - 1)) && n != 20 && n != 40) return HQMQ_ERR_SHAPE;
    if (a->idx_bits < 1 || a->idx_bits > 16 || a->aux_bits < 0 || a->aux_bits > 8) return HQMQ_ERR_LAYOUT;
    if ((a->K.flag_plane != nullptr) != (a->V.flag_plane != nullptr)) return HQMQ_ERR_NULL;
    const bool flags = a->K.flag_plane != nullptr;
    if (flags && n > 32) return HQMQ_ERR_SHAPE;
    const int elt = a->dtype == HQMQ_F32 ? 4 : 2;
    if (((uintptr_t)a->Q % (4 * elt)) || (a->q_sb % 4) || (a->q_sh % 4) || (a->q_st % 4)) return HQMQ_ERR_ALIGN;
    if (((uintptr_t)a->K.joint % (4 * elt)) || ((uintptr_t)a->V.joint % (4 * elt))) return HQMQ_ERR_ALIGN;
    if (((uintptr_t)a->K.main_plane & 15) || ((uintptr_t)a->V.main_plane & 15)) return HQMQ_ERR_ALIGN;
    if (flags && (((uintptr_t)a->K.sideband % (4 * elt)) || ((uintptr_t)a->V.sideband % (4 * elt)))) return HQMQ_ERR_ALIGN;

    int n_splits = a->n_splits > 0 ? a->n_splits : hqmq_attn_pick_splits(a->B, a->H_q, a->H_kv, a->T_q, a->T_kv, a->kv_len != nullptr);
    if (n_splits > 8192) return HQMQ_ERR_SHAPE;   // bound of hqmq_attn_combine
    if (n_splits > 1) {
        if (!a->workspace) return HQMQ_ERR_NULL;
        if (a->workspace_bytes < hqmq_attn_workspace_bytes(a->B, a->H_q, a->T_q, 4 * n, n_splits)) return HQMQ_ERR_WORKSPACE;
        if ((uintptr_t)a->workspace & 15) return HQMQ_ERR_ALIGN;
    }
    // LDS: the two fp16 codeword tables, reused afterwards for the cross-wave merge
    size_t shmem = ((size_t)a->K.K + a->V.K) * 8;
    const size_t merge = (size_t)kAttnWaves * 16 * (4 * n + 2) * sizeof(float);
    if (shmem < merge) shmem = merge;
    if (shmem > 152 * 1024) return HQMQ_ERR_SHAPE;

    AttnParams p;
    p.Q = a->Q; p.O = a->O;
    p.qsb = a->q_sb; p.qsh = a->q_sh; p.qst = a->q_st; p.osb = a->o_sb; p.osh = a->o_sh; p.ost = a->o_st;
    p.Kc = to_dev(a->K); p.Vc = to_dev(a->V);
    p.dtype = a->dtype;
    p.B = a->B; p.Hq = a->H_q; p.Hkv = a->H_kv; p.G = a->H_q / a->H_kv; p.Tq = a->T_q; p.Tkv = a->T_kv; p.n = n;
    p.t_cap = a->t_cap;
    p.idx_bits = a->idx_bits; p.aux_bits = a->aux_bits; p.qmax = a->qmax;
    p.kv_len = a->kv_len; p.kv_start = a->kv_start; p.batch_order = a->batch_order; p.causal = a->causal; p.causal_offset = a->causal_offset;
    p.c_log2 = a->softmax_scale * 1.4426950408889634f / (float)a->qmax;
    p.c_plain = a->softmax_scale * 1.4426950408889634f;
    p.inv_qmax = 1.0f / (float)a->qmax;
    p.n_splits = n_splits;
    p.n_cg = (a->T_q * p.G + 15) / 16;
    p.ws = (float *)a->workspace;
    // Workgroups go to the eight XCDs round-robin in dispatch order.  Numbering them (sequence, KV head)-fastest puts
    // all blocks of one KV head on one XCD, whose L2 then fetches that head's two codeword tables once for all of them.
    // Ragged batches keep the sequence-major order that batch_order relies on.
    p.xcd_remap = (!a->kv_len && !a->batch_order && ((a->B * a->H_kv) % 8) == 0) ? 1 : 0;
    p.tab_fp8 = a->fp8_table_storage ? 1 : 0;
    p.wide_range = a->wide_range ? 1 : 0;
    p.no_lds_landing = a->force_generic == 2 ? 1 : 0;
    // 4 consecutive scales with one vector load: unit stride, aligned rows, and capacity rows readable
    const int salign = a->dtype == HQMQ_F32 ? 16 : 8;
    p.scale_vec = 1;
    for (const hqmq_packed *k : pk)
        if (k->scale_st != 1 || (k->scale_sb % 4) || (k->scale_sh % 4) || ((uintptr_t)k->scale_plane % salign) ||
            k->scale_sh < a->t_cap || (a->t_cap % kSuper))
            p.scale_vec = 0;
    if (p.n_cg > 65535) return HQMQ_ERR_SHAPE;
    dim3 grid((unsigned)n_splits, (unsigned)p.n_cg, (unsigned)(a->B * a->H_kv));
    {
        const uint64_t gx = grid.x, gy = grid.y, gz = grid.z;
        p.m_gz = attn_div_magic(gz, gx * gy * gz);
        p.m_gx = attn_div_magic(gx, gx * gy);
        p.m_hkv = attn_div_magic((uint64_t)a->H_kv, gz);
        p.m_G = attn_div_magic((uint64_t)p.G, gy * 16);
        p.m_splits = attn_div_magic((uint64_t)n_splits, (uint64_t)a->T_kv + (uint64_t)n_splits);
        if ((gz > 1 && !p.m_gz) || (gx > 1 && !p.m_gx)) p.xcd_remap = 0;      // no multiplier for the renumbering: keep the grid order
    }
    hipStream_t st = (hipStream_t)stream;
    LaunchTiming tm;
    tm.start = (hipEvent_t)a->start_event;
    tm.stop = (hipEvent_t)a->stop_event;
    int rc = HQMQ_OK;
    bool handled = false;
    if (p.scale_vec && a->force_generic != 1 && a->softmax_scale > 0.f) {
        rc = launch_attn_fast(p, a->main_bits, flags, grid, ((size_t)a->K.K + a->V.K) * 8, st, tm, &handled);
        if (rc) return rc;
    }
    if (!handled) switch (n / 4) {
        case 1: rc = launch_attn_mb<1>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        case 2: rc = launch_attn_mb<2>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        case 4: rc = launch_attn_mb<4>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        case 5: rc = launch_attn_mb<5>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        case 8: rc = launch_attn_mb<8>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        case 10: rc = launch_attn_mb<10>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        case 16: rc = launch_attn_mb<16>(p, a->main_bits, flags, grid, shmem, st, tm); break;
        default: return HQMQ_ERR_SHAPE;
    }
    if (rc) return rc;
    if (n_splits > 1 && !a->skip_combine)
        rc = hqmq_attn_combine(a->workspace, a->O, a->dtype, a->B, a->H_q, a->T_q, 4 * n, n_splits, a->o_sb, a->o_sh, a->o_st,
                               stream);
    return rc;
}

extern "C" int hqmq_attn_fwd(const hqmq_attn_args *a, void *stream) { return attn_fwd_impl(a, stream); }

// ---- the entry point that allocates nothing: split partials in a static device array ----
// Every GPU the library runs on holds its own copy of this array at its own address until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; kernels and host calls use the
// per-device address looked up below.
static __device__ __align__(256) unsigned char scratch[HQMQ_ATTN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// The device address of `scratch` on the current device; looked up once per device.
int static_scratch(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HQMQ_ERR_SHAPE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return HQMQ_ERR_NULL;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return HQMQ_OK;
}
}  // namespace

extern "C" int64_t hqmq_attn_static_scratch_bytes(void) { return HQMQ_ATTN_STATIC_SCRATCH_BYTES; }

extern "C" int hqmq_attn_fwd_static(const hqmq_attn_args *a, void *stream) {
    if (!a) return HQMQ_ERR_NULL;
    if (a->skip_combine) return HQMQ_ERR_SCRATCH;       // the partials would stay in memory the caller cannot name
    if (a->B < 1 || a->H_q < 1 || a->H_kv < 1 || a->T_q < 1 || a->T_kv < 0 || a->n_chunks < 1) return HQMQ_ERR_SHAPE;
    hqmq_attn_args b = *a;
    b.n_splits = a->n_splits > 0 ? a->n_splits : hqmq_attn_pick_splits(a->B, a->H_q, a->H_kv, a->T_q, a->T_kv, a->kv_len != nullptr);
    if (b.n_splits > 8192) return HQMQ_ERR_SHAPE;
    b.workspace = nullptr;
    b.workspace_bytes = 0;
    if (b.n_splits > 1) {
        // the partials of this call, (m, l, acc) per (row, split), are all written before they are read:
        // nothing in the array has to start at zero
        const int64_t need = hqmq_attn_workspace_bytes(a->B, a->H_q, a->T_q, 4 * a->n_chunks, b.n_splits);
        if (need > (int64_t)HQMQ_ATTN_STATIC_SCRATCH_BYTES) return HQMQ_ERR_SCRATCH;
        void *ptr = nullptr;
        const int rc = static_scratch(&ptr);
        if (rc) return rc;
        b.workspace = ptr;
        b.workspace_bytes = HQMQ_ATTN_STATIC_SCRATCH_BYTES;
    }
    return attn_fwd_impl(&b, stream);
}
