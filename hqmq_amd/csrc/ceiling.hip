// Measurement aid: a kernel that only READS the planes of a packed cache, with the grid, the per-wavefront token
// half-steps and the per-lane load pattern of the specialised decode-attention kernel (16-byte loads of the main
// rows of K and V, 8-byte loads of four scales, 32 tokens per step), and a ring of DEPTH such steps in flight.
// Its duration is what the memory system allows a kernel of this shape; the attention kernel's distance from it
// is what its own arithmetic, tables and merge cost.  Supports the 16+0 layout at d_h = 128 (s96_r4), no sideband.
#include "attention_common.h"

namespace hqmq {

struct StepWords {
    uint4 k[2], v[2];
    uint2 ks[2], vs[2];
};

template <int DEPTH, int WV>
__global__ __launch_bounds__(WV * 64) void read_ceiling_kernel(const uint8_t *kmain, const uint8_t *vmain, const uint16_t *kscale,
                                                              const uint16_t *vscale, int64_t t_cap, int Tkv, int n_splits,
                                                              int nbh, int remap, uint32_t *sink) {
    int sp = blockIdx.x, bh = blockIdx.z;
    if (remap) {        // (sequence, KV head) fastest, as the attention kernel numbers its blocks
        const unsigned lin = blockIdx.x + gridDim.x * blockIdx.z;
        sp = (int)(lin / (unsigned)nbh);
        bh = (int)(lin - (unsigned)sp * (unsigned)nbh);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, grp = lane >> 4;
    int per_split = (Tkv + n_splits - 1) / n_splits;
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int b_begin = min(sp * per_split, Tkv), b_end = min(Tkv, b_begin + per_split);
    // half-steps round-robin over the block's wavefronts, as in the attention kernel
    constexpr int STRIDE = 32 * WV;
    const int t_begin = min(b_begin + wave * 32, b_end), t_end = b_end;
    constexpr int mrb = 64;
    const uint8_t *k_rows = kmain + (size_t)bh * t_cap * mrb + col * mrb + grp * 16;
    const uint8_t *v_rows = vmain + (size_t)bh * t_cap * mrb + col * mrb + grp * 16;
    const uint16_t *ks = kscale + (size_t)bh * t_cap + 4 * grp, *vs = vscale + (size_t)bh * t_cap + 4 * grp;
    auto load = [&](int t, StepWords &w) {
        t = min(t, (int)t_cap - 32);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            w.k[u] = *reinterpret_cast<const uint4 *>(k_rows + (size_t)(t + 16 * u) * mrb);
            w.ks[u] = *reinterpret_cast<const uint2 *>(ks + t + 16 * u);
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            w.v[u] = *reinterpret_cast<const uint4 *>(v_rows + (size_t)(t + 16 * u) * mrb);
            w.vs[u] = *reinterpret_cast<const uint2 *>(vs + t + 16 * u);
        }
    };
    uint32_t acc = 0;
    auto consume = [&](const StepWords &w) {
#pragma unroll
        for (int u = 0; u < 2; u++)
            acc ^= w.k[u].x ^ w.k[u].y ^ w.k[u].z ^ w.k[u].w ^ w.v[u].x ^ w.v[u].y ^ w.v[u].z ^ w.v[u].w ^ w.ks[u].x ^ w.ks[u].y ^
                   w.vs[u].x ^ w.vs[u].y;
    };
    StepWords ring[DEPTH];
    if (t_begin < t_end) {
#pragma unroll
        for (int d = 0; d < DEPTH - 1; d++) load(t_begin + STRIDE * d < t_end ? t_begin + STRIDE * d : t_begin, ring[d]);
        int t = t_begin;
        while (true) {
            bool done = false;
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                const int tn = t + STRIDE * (DEPTH - 1);
                load(tn < t_end ? tn : t, ring[(d + DEPTH - 1) % DEPTH]);
                consume(ring[d]);
                t += STRIDE;
                if (t >= t_end) { done = true; break; }
            }
            if (done) break;
        }
    }
    sink[((size_t)blockIdx.z * gridDim.x + blockIdx.x) * (WV * 64) + threadIdx.x] = acc;
}

template <int DEPTH>
static int launch_depth(int waves, dim3 grid, hipStream_t st, const LaunchTiming &tm, const uint8_t *km, const uint8_t *vm,
                        const uint16_t *ks, const uint16_t *vs, int64_t t_cap, int Tkv, int n_splits, int nbh, int remap, uint32_t *sink) {
    if (waves == 12) {
        auto kern = read_ceiling_kernel<DEPTH, 12>;
        if (tm.start || tm.stop) hipExtLaunchKernelGGL(kern, grid, dim3(768), 0, st, tm.start, tm.stop, 0, km, vm, ks, vs, t_cap, Tkv, n_splits, nbh, remap, sink);
        else hipLaunchKernelGGL(kern, grid, dim3(768), 0, st, km, vm, ks, vs, t_cap, Tkv, n_splits, nbh, remap, sink);
    } else {
        auto kern = read_ceiling_kernel<DEPTH, 8>;
        if (tm.start || tm.stop) hipExtLaunchKernelGGL(kern, grid, dim3(512), 0, st, tm.start, tm.stop, 0, km, vm, ks, vs, t_cap, Tkv, n_splits, nbh, remap, sink);
        else hipLaunchKernelGGL(kern, grid, dim3(512), 0, st, km, vm, ks, vs, t_cap, Tkv, n_splits, nbh, remap, sink);
    }
    return hip_status(hipGetLastError());
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int64_t hqmq_attn_read_ceiling_sink_bytes(int B, int H_kv, int n_splits) {
    return (int64_t)B * H_kv * n_splits * 768 * 4;
}

extern "C" int hqmq_attn_read_ceiling(const hqmq_attn_args *a, int depth, int waves, void *sink, int64_t sink_bytes, void *stream) {
    if (!a || !sink || !a->K.main_plane || !a->V.main_plane || !a->K.scale_plane || !a->V.scale_plane) return HQMQ_ERR_NULL;
    if (a->dtype != HQMQ_F16 && a->dtype != HQMQ_BF16) return HQMQ_ERR_DTYPE;
    if (a->n_chunks != 32 || a->main_bits != 16 || a->aux_bits != 0 || a->K.flag_plane || a->V.flag_plane) return HQMQ_ERR_LAYOUT;
    if (a->B < 1 || a->H_kv < 1 || a->T_kv < 1 || a->t_cap < a->T_kv || (a->t_cap % kSuper) || (int64_t)a->B * a->H_kv > 65535) return HQMQ_ERR_SHAPE;
    if (a->K.scale_st != 1 || a->V.scale_st != 1 || a->K.scale_sh != a->t_cap || a->V.scale_sh != a->t_cap ||
        a->K.scale_sb != a->t_cap * a->H_kv || a->V.scale_sb != a->t_cap * a->H_kv) return HQMQ_ERR_SHAPE;
    if (waves != 8 && waves != 12) return HQMQ_ERR_SHAPE;
    const int n_splits = a->n_splits > 0 ? a->n_splits : hqmq_attn_pick_splits(a->B, a->H_q, a->H_kv, 1, a->T_kv, 0);
    if (sink_bytes < hqmq_attn_read_ceiling_sink_bytes(a->B, a->H_kv, n_splits)) return HQMQ_ERR_WORKSPACE;
    const int nbh = a->B * a->H_kv;
    dim3 grid((unsigned)n_splits, 1, (unsigned)nbh);
    LaunchTiming tm;
    tm.start = (hipEvent_t)a->start_event;
    tm.stop = (hipEvent_t)a->stop_event;
    const int remap = (nbh % 8) == 0;
    const uint8_t *km = a->K.main_plane, *vm = a->V.main_plane;
    const uint16_t *ks = (const uint16_t *)a->K.scale_plane, *vs = (const uint16_t *)a->V.scale_plane;
    hipStream_t st = (hipStream_t)stream;
    switch (depth) {
        case 2: return launch_depth<2>(waves, grid, st, tm, km, vm, ks, vs, a->t_cap, a->T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        case 3: return launch_depth<3>(waves, grid, st, tm, km, vm, ks, vs, a->t_cap, a->T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        case 4: return launch_depth<4>(waves, grid, st, tm, km, vm, ks, vs, a->t_cap, a->T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        case 6: return launch_depth<6>(waves, grid, st, tm, km, vm, ks, vs, a->t_cap, a->T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        default: return HQMQ_ERR_SHAPE;
    }
}
