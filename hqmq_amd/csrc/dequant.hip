// Dense decode kernels and the code packer.
//   hqmq_dequant         unpacked codes -> dense, rounding of _decode_kv_torch
//                        (src/quantizers/hqmq_attention.py:39-65 of the reference);
//                        replaces hqmq_decode_triton (src/quantizers/hqmq_kernel.py:102-132)
//   hqmq_pack_codes      unpacked int32 codes -> packed main/aux rows
//   hqmq_dequant_packed  packed cache (+ outlier sideband) -> dense
// Compiled with -ffp-contract=off: every product rounds to D on its own.
#include "common.h"

namespace hqmq {

// bits [bitpos, bitpos+nbits) of a little-endian bit stream held in `row` (row_bytes long)
__device__ __forceinline__ uint32_t read_bits(const uint8_t *row, int row_bytes, int bitpos, int nbits) {
    uint32_t v = 0;
    int byte = bitpos >> 3, sh = bitpos & 7, got = 0;
    while (got < nbits && byte < row_bytes) {
        v |= ((uint32_t)row[byte] >> sh) << got;
        got += 8 - sh;
        sh = 0;
        byte++;
    }
    return nbits >= 32 ? v : (v & ((1u << nbits) - 1u));
}

template <class D>
__global__ void dequant_kernel(const int32_t *idx, int64_t isb, int64_t ish, int64_t ist, const int32_t *rq, int64_t rsb_,
                               int64_t rsh_, int64_t rst_, const typename D::storage *rs, int64_t ssb, int64_t ssh,
                               int64_t sst, const typename D::storage *joint, int64_t jsh, int K, int B, int H, int T, int n,
                               int qmax, typename D::storage *out) {
    const int64_t total = (int64_t)B * H * T * n;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(g % n);
        const int64_t row = g / n;
        const int t = (int)(row % T);
        const int h = (int)((row / T) % H);
        const int b = (int)(row / ((int64_t)T * H));
        int k = idx[b * isb + h * ish + t * ist + c];
        k = k < 0 ? 0 : (k >= K ? K - 1 : k);
        const float q = D::rnd((float)rq[b * rsb_ + h * rsh_ + t * rst_ + c]);
        const float s = D::load(rs + b * ssb + h * ssh + t * sst);
        const float r = D::rnd(D::rnd(q * s) / (float)qmax);
        const typename D::storage *cw = joint + h * jsh + (int64_t)k * 4;
        for (int j = 0; j < 4; j++) D::store(out + g * 4 + j, D::rnd(D::load(cw + j) * r));
    }
}

// one thread per output byte of the main plane, then of the aux plane
__global__ void pack_codes_kernel(const int32_t *idx, int64_t isb, int64_t ish, int64_t ist, const int32_t *rq, int64_t rsb_,
                                  int64_t rsh_, int64_t rst_, int B, int H, int T, int n, int idx_bits, int main_bits,
                                  int aux_bits, uint8_t *main_plane, uint8_t *aux_plane, int64_t t_cap) {
    const int mrb = (n * main_bits + 7) >> 3, arb = (n * aux_bits + 7) >> 3;
    const int per_row = mrb + arb;
    const int64_t total = (int64_t)B * H * T * per_row;
    const uint32_t idx_mask = (1u << idx_bits) - 1u;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        int byte = (int)(g % per_row);
        const int64_t row = g / per_row;
        const int t = (int)(row % T);
        const int h = (int)((row / T) % H);
        const int b = (int)(row / ((int64_t)T * H));
        const bool is_aux = byte >= mrb;
        if (is_aux) byte -= mrb;
        const int w = is_aux ? aux_bits : main_bits, shift = is_aux ? main_bits : 0;
        const int32_t *ip = idx + b * isb + h * ish + t * ist;
        const int32_t *rp = rq + b * rsb_ + h * rsh_ + t * rst_;
        uint32_t outv = 0;
        for (int bit = 0; bit < 8; bit++) {
            const int pos = byte * 8 + bit, i = pos / w, o = pos - i * w;
            if (i < n) {
                const uint32_t code = ((uint32_t)ip[i] & idx_mask) | ((uint32_t)rp[i] << idx_bits);
                outv |= ((((code >> shift) & ((1u << w) - 1u)) >> o) & 1u) << bit;
            }
        }
        const size_t prow = ((size_t)b * H + h) * t_cap + t;
        if (is_aux) aux_plane[prow * arb + byte] = (uint8_t)outv;
        else main_plane[prow * mrb + byte] = (uint8_t)outv;
    }
}

struct PackedView {
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

// mode 0: value = cw * ((rq * rs) / qmax)   (the attention kernels' convention)
// mode 1: value = (rq * (rs / qmax)) * cw   (the quantizer's fake-quant output)
template <class D>
__global__ void dequant_packed_kernel(PackedView p, int B, int H, int T, int n, int64_t t_cap, int idx_bits, int main_bits,
                                      int aux_bits, int qmax, int mode, typename D::storage *out) {
    using ST = typename D::storage;
    const int mrb = (n * main_bits + 7) >> 3, arb = (n * aux_bits + 7) >> 3, frb = (n + 7) >> 3;
    const int64_t total = (int64_t)B * H * T * n;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(g % n);
        const int64_t row = g / n;
        const int t = (int)(row % T);
        const int h = (int)((row / T) % H);
        const int b = (int)(row / ((int64_t)T * H));
        const size_t bh = (size_t)b * H + h;
        const size_t prow = bh * t_cap + t;
        ST *dst = out + g * 4;
        if (p.flag_plane && ((p.flag_plane[prow * frb + (c >> 3)] >> (c & 7)) & 1)) {
            const int tile = t >> 4;
            // 64-bit and clamped on both sides: a tile that was never written (or was cropped) holds INT32_MAX
            int64_t rank = p.sb_tile_off[bh * ((t_cap + kTile - 1) / kTile) + tile];
            for (int tt = tile * kTile; tt < t; tt++)
                for (int by = 0; by < frb; by++) rank += __popc((uint32_t)p.flag_plane[(bh * t_cap + tt) * frb + by]);
            for (int cc = 0; cc < c; cc++) rank += (p.flag_plane[prow * frb + (cc >> 3)] >> (cc & 7)) & 1;
            rank = rank < 0 ? 0 : (rank < p.sb_cap ? rank : p.sb_cap - 1);
            const ST *src = (const ST *)p.sideband + (bh * p.sb_cap + rank) * 4;
            for (int j = 0; j < 4; j++) dst[j] = src[j];
            continue;
        }
        uint32_t code = read_bits(p.main_plane + prow * mrb, mrb, c * main_bits, main_bits);
        if (aux_bits) code |= read_bits(p.aux_plane + prow * arb, arb, c * aux_bits, aux_bits) << main_bits;
        int k = (int)(code & ((1u << idx_bits) - 1u));
        k = k >= p.K ? p.K - 1 : k;
        const float q = (float)(code >> idx_bits);
        const float s = D::load((const ST *)p.scale_plane + b * p.ssb + h * p.ssh + t * p.sst);
        const ST *cw = (const ST *)p.joint + h * p.jsh + (int64_t)k * 4;
        if (mode == 0) {
            const float r = D::rnd(D::rnd(D::rnd(q) * s) / (float)qmax);
            for (int j = 0; j < 4; j++) D::store(dst + j, D::rnd(D::load(cw + j) * r));
        } else {
            const float r = D::rnd(q * D::rnd(s / (float)qmax));
            for (int j = 0; j < 4; j++) D::store(dst + j, D::rnd(r * D::load(cw + j)));
        }
    }
}

static inline int grid_for(int64_t total, int block) {
    int64_t g = (total + block - 1) / block;
    return (int)(g < 1 ? 1 : (g > 65535 * 16 ? 65535 * 16 : g));
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int hqmq_dequant(const int32_t *idx, int64_t idx_sb, int64_t idx_sh, int64_t idx_st, const int32_t *rq,
                            int64_t rq_sb, int64_t rq_sh, int64_t rq_st, const void *rs, int64_t rs_sb, int64_t rs_sh,
                            int64_t rs_st, const void *joint, int64_t joint_sh, int K, int dtype, int B, int H, int T,
                            int n_chunks, int qmax, void *out, void *stream) {
    if (!idx || !rq || !rs || !joint || !out) return HQMQ_ERR_NULL;
    if (B < 1 || H < 1 || T < 0 || n_chunks < 1 || K < 1 || qmax < 1) return HQMQ_ERR_SHAPE;
    if (T == 0) return HQMQ_OK;
    const int64_t total = (int64_t)B * H * T * n_chunks;
    dim3 grid(grid_for(total, 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(DT, ST)                                                                                                   \
    hipLaunchKernelGGL(dequant_kernel<DT>, grid, block, 0, st, idx, idx_sb, idx_sh, idx_st, rq, rq_sb, rq_sh, rq_st,      \
                       (const ST *)rs, rs_sb, rs_sh, rs_st, (const ST *)joint, joint_sh, K, B, H, T, n_chunks, qmax, (ST *)out)
    switch (dtype) {
        case HQMQ_F32: LAUNCH(F32, float); break;
        case HQMQ_F16: LAUNCH(F16, uint16_t); break;
        case HQMQ_BF16: LAUNCH(BF16, uint16_t); break;
        default: return HQMQ_ERR_DTYPE;
    }
#undef LAUNCH
    return hip_status(hipGetLastError());
}

extern "C" int hqmq_pack_codes(const int32_t *idx, int64_t idx_sb, int64_t idx_sh, int64_t idx_st, const int32_t *rq,
                               int64_t rq_sb, int64_t rq_sh, int64_t rq_st, int B, int H, int T, int n_chunks, int idx_bits,
                               int main_bits, int aux_bits, uint8_t *main_plane, uint8_t *aux_plane, int64_t t_cap,
                               void *stream) {
    if (!idx || !rq || !main_plane || (aux_bits && !aux_plane)) return HQMQ_ERR_NULL;
    if (B < 1 || H < 1 || T < 0 || n_chunks < 1 || t_cap < T) return HQMQ_ERR_SHAPE;
    if (idx_bits < 1 || idx_bits > 16 || main_bits < 1 || main_bits > 16 || aux_bits < 0 || aux_bits > 8) return HQMQ_ERR_LAYOUT;
    if (T == 0) return HQMQ_OK;
    const int per_row = ((n_chunks * main_bits + 7) >> 3) + ((n_chunks * aux_bits + 7) >> 3);
    dim3 grid(grid_for((int64_t)B * H * T * per_row, 256)), block(256);
    hipLaunchKernelGGL(pack_codes_kernel, grid, block, 0, (hipStream_t)stream, idx, idx_sb, idx_sh, idx_st, rq, rq_sb, rq_sh,
                       rq_st, B, H, T, n_chunks, idx_bits, main_bits, aux_bits, main_plane, aux_plane, t_cap);
    return hip_status(hipGetLastError());
}

extern "C" int hqmq_dequant_packed(const hqmq_packed *p, int dtype, int B, int H, int T, int n_chunks, int64_t t_cap,
                                   int idx_bits, int main_bits, int aux_bits, int qmax, int mode, void *out, void *stream) {
    if (!p || !p->main_plane || !p->scale_plane || !p->joint || !out) return HQMQ_ERR_NULL;
    if (aux_bits && !p->aux_plane) return HQMQ_ERR_NULL;
    if (p->flag_plane && (!p->sideband || !p->sb_tile_off || p->sb_cap < 1)) return HQMQ_ERR_NULL;
    if (B < 1 || H < 1 || T < 0 || n_chunks < 1 || t_cap < T || qmax < 1) return HQMQ_ERR_SHAPE;
    if (mode != 0 && mode != 1) return HQMQ_ERR_SHAPE;
    if (T == 0) return HQMQ_OK;
    PackedView v{p->main_plane, p->aux_plane, p->flag_plane, p->scale_plane, p->scale_sb, p->scale_sh, p->scale_st,
                 p->sideband, p->sb_tile_off, p->sb_cap, p->joint, p->joint_sh, p->K};
    dim3 grid(grid_for((int64_t)B * H * T * n_chunks, 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(DT, ST)                                                                                                  \
    hipLaunchKernelGGL(dequant_packed_kernel<DT>, grid, block, 0, st, v, B, H, T, n_chunks, t_cap, idx_bits, main_bits, \
                       aux_bits, qmax, mode, (ST *)out)
    switch (dtype) {
        case HQMQ_F32: LAUNCH(F32, float); break;
        case HQMQ_F16: LAUNCH(F16, uint16_t); break;
        case HQMQ_BF16: LAUNCH(BF16, uint16_t); break;
        default: return HQMQ_ERR_DTYPE;
    }
#undef LAUNCH
    return hip_status(hipGetLastError());
}
