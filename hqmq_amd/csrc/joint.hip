// Joint codebook q_p * q_s in D with op-by-op rounding (k = p*S + s), plus the
// per-head rounding slack the quantize kernel's candidate filter relies on.
// Follows HQMQQuantizer._get_codebook (src/quantizers/hqmq.py:119-143) and
// _make_24cell_codebook (src/quantizers/spherical.py:22-43) of the reference.
// Compiled with -ffp-contract=off: every written operation rounds on its own.
#include "common.h"

namespace hqmq {

__device__ __forceinline__ void cell24_vertex(int p, float v[4]) {
    if (p < 8) {
        for (int j = 0; j < 4; j++) v[j] = (j == (p >> 1)) ? ((p & 1) ? -1.0f : 1.0f) : 0.0f;
    } else {
        int m = p - 8;
        for (int j = 0; j < 4; j++) v[j] = ((m >> (3 - j)) & 1) ? -0.5f : 0.5f;
    }
}

template <class D>
__device__ __forceinline__ void quat_mul_d(const float a[4], const float b[4], float o[4]) {
    auto M = [](float x, float y) { return D::rnd(x * y); };
    auto A = [](float x, float y) { return D::rnd(x + y); };
    auto S = [](float x, float y) { return D::rnd(x - y); };
    o[0] = S(S(S(M(a[0], b[0]), M(a[1], b[1])), M(a[2], b[2])), M(a[3], b[3]));
    o[1] = S(A(A(M(a[0], b[1]), M(a[1], b[0])), M(a[2], b[3])), M(a[3], b[2]));
    o[2] = A(A(S(M(a[0], b[2]), M(a[1], b[3])), M(a[2], b[0])), M(a[3], b[1]));
    o[3] = A(S(A(M(a[0], b[3]), M(a[1], b[2])), M(a[2], b[1])), M(a[3], b[0]));
}

// One block per head.
template <class D>
__global__ void build_joint_kernel(const float *__restrict__ raw, int S, typename D::storage *__restrict__ joint,
                                   float *__restrict__ slack) {
    const int h = blockIdx.x;
    __shared__ float red[256];
    float worst = 0.f;
    for (int s = threadIdx.x; s < S; s += blockDim.x) {
        const float *r = raw + ((size_t)h * S + s) * 4;
        float nrm = norm4(r[0], r[1], r[2], r[3]);
        if (!is_nan(nrm) && nrm < 1e-8f) nrm = 1e-8f;
        float q[4];
        for (int j = 0; j < 4; j++) q[j] = D::rnd(r[j] / nrm);
        for (int p = 0; p < 24; p++) {
            float pv[4], o[4];
            cell24_vertex(p, pv);
            quat_mul_d<D>(pv, q, o);
            // exact product of the same operands, in double
            double a0 = pv[0], a1 = pv[1], a2 = pv[2], a3 = pv[3];
            double b0 = q[0], b1 = q[1], b2 = q[2], b3 = q[3];
            double e0 = a0 * b0 - a1 * b1 - a2 * b2 - a3 * b3;
            double e1 = a0 * b1 + a1 * b0 + a2 * b3 - a3 * b2;
            double e2 = a0 * b2 - a1 * b3 + a2 * b0 + a3 * b1;
            double e3 = a0 * b3 + a1 * b2 - a2 * b1 + a3 * b0;
            double d0 = o[0] - e0, d1 = o[1] - e1, d2 = o[2] - e2, d3 = o[3] - e3;
            float err = (float)sqrt(d0 * d0 + d1 * d1 + d2 * d2 + d3 * d3);
            if (err > worst || is_nan(err)) worst = err;
            typename D::storage *dst = joint + (((size_t)h * 24 + p) * S + s) * 4;
            for (int j = 0; j < 4; j++) D::store(dst + j, o[j]);
        }
    }
    red[threadIdx.x] = worst;
    __syncthreads();
    for (int w = blockDim.x / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) {
            float o = red[threadIdx.x + w];
            if (o > red[threadIdx.x] || is_nan(o)) red[threadIdx.x] = o;
        }
        __syncthreads();
    }
    // a hair above the measured maximum covers the float rounding of `err` itself
    if (threadIdx.x == 0 && slack) slack[h] = red[0] * 1.0001f + 1e-9f;
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int hqmq_build_joint(const float *raw, int H, int S, int dtype, void *joint, float *slack, void *stream) {
    if (!raw || !joint) return HQMQ_ERR_NULL;
    if (H < 1 || S < 1 || S > 2730) return HQMQ_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(H), block(256);
    switch (dtype) {
        case HQMQ_F32: hipLaunchKernelGGL(build_joint_kernel<F32>, grid, block, 0, st, raw, S, (float *)joint, slack); break;
        case HQMQ_F16: hipLaunchKernelGGL(build_joint_kernel<F16>, grid, block, 0, st, raw, S, (uint16_t *)joint, slack); break;
        case HQMQ_BF16: hipLaunchKernelGGL(build_joint_kernel<BF16>, grid, block, 0, st, raw, S, (uint16_t *)joint, slack); break;
        default: return HQMQ_ERR_DTYPE;
    }
    return hip_status(hipGetLastError());
}
