// Shared device helpers for the HQMQ kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/hqmq_amd.h"

#define HQMQ_VERSION 0x000200  // 0x000200: hqmq_packed gained scale_max_bits (every struct that embeds it moved), partial records are d_h + 4 floats, the read probes left the library

namespace hqmq {

constexpr int kWave = 64;
constexpr int kTile = 16;  // tokens per sideband tile / MFMA tile

// ---- bit-exact conversions: fp32 <-> D with round-to-nearest-even ----------
struct F32 {
    using storage = float;
    static constexpr int code = HQMQ_F32;
    static __device__ __forceinline__ float load(const storage *p) { return *p; }
    static __device__ __forceinline__ void store(storage *p, float f) { *p = f; }
    static __device__ __forceinline__ float rnd(float f) { return f; }
    static __device__ __forceinline__ float eps() { return 5.9604645e-8f; }  // 2^-24
};
struct F16 {
    using storage = uint16_t;
    static constexpr int code = HQMQ_F16;
    static __device__ __forceinline__ float load(const storage *p) { return __half2float(__ushort_as_half(*p)); }
    static __device__ __forceinline__ void store(storage *p, float f) { *p = __half_as_ushort(__float2half_rn(f)); }
    // The empty asm keeps the fp32 value opaque: without it the compiler folds a preceding fused
    // multiply-add into v_fma_mixlo_f16, which rounds once to fp16 instead of fp32-then-fp16.
    static __device__ __forceinline__ float rnd(float f) {
        asm volatile("" : "+v"(f));
        return __half2float(__float2half_rn(f));
    }
    static __device__ __forceinline__ float eps() { return 4.8828125e-4f; }  // 2^-11
};
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}
struct BF16 {
    using storage = uint16_t;
    static constexpr int code = HQMQ_BF16;
    static __device__ __forceinline__ float load(const storage *p) { return __uint_as_float((uint32_t)(*p) << 16); }
    static __device__ __forceinline__ void store(storage *p, float f) { *p = f32_to_bf16_bits(f); }
    static __device__ __forceinline__ float rnd(float f) { return __uint_as_float((uint32_t)f32_to_bf16_bits(f) << 16); }
    static __device__ __forceinline__ float eps() { return 3.90625e-3f; }  // 2^-8
};

__device__ __forceinline__ bool is_nan(float f) { return f != f; }

// torch clamp(min=c) on a D tensor: NaN propagates, the bound is rounded to D.
template <class D>
__device__ __forceinline__ float clamp_min_d(float v, float lo_f32) {
    if (is_nan(v)) return v;
    float lo = D::rnd(lo_f32);
    return v < lo ? lo : v;
}

// ||chunk||_2 as torch's CPU norm computes it: fp32, products and sums rounded one by one.
// Built with -ffp-contract=off, so none of these fuse.
__device__ __forceinline__ float norm4(float a, float b, float c, float d) {
    float s = a * a;
    s = s + b * b;
    s = s + c * c;
    s = s + d * d;
    return sqrtf(s);
}

inline int layout_bits(int S, int radius_bits, int *idx_bits, int *main_bits, int *aux_bits) {
    if (S < 1 || S > 2730 || radius_bits < 1 || radius_bits > 8) return HQMQ_ERR_SHAPE;
    int K = 24 * S, ib = 0;
    while ((1 << ib) < K) ib++;
    int cb = ib + radius_bits;
    int mb = 4 * (cb / 4);
    if (mb < 8) mb = 8;
    if (mb > 16) mb = 16;
    int ab = cb > mb ? cb - mb : 0;
    if (idx_bits) *idx_bits = ib;
    if (main_bits) *main_bits = mb;
    if (aux_bits) *aux_bits = ab;
    return HQMQ_OK;
}

inline int hip_status(hipError_t e) { return e == hipSuccess ? HQMQ_OK : (int)e; }

// ---- the stages of an append, for one tensor or for the K and the V tensor of a cache together ----
// With two calls of equal shape every stage is one launch whose blocks split between the tensors; otherwise the
// calls run one after the other.  Results are those of the single-tensor entry points either way.
struct Med3xCall {
    const void *x; int64_t xsb, xsh, xst;
    int dtype, B, H, T, n;
    float mult;
    void *ws; int64_t ws_bytes;
    float *median; void *thr; int32_t *n_out;
};
struct CompactCall {
    const void *x; int64_t xsb, xsh, xst;
    int dtype, B, H, T, n;
    const uint8_t *flag_plane; int64_t t_cap; int t_off; const int32_t *pos;
    void *sideband; int64_t sb_cap; int32_t *sb_tile_off, *sb_count, *overflow; uint16_t *sb_coord;
    // the packed planes of the same rows (main_plane NULL: none).  With them a flagged chunk that finds the sideband
    // full is turned back into a plain chunk (flag bit cleared, its radius code written) instead of decoding to zero.
    uint8_t *main_plane, *aux_plane; const void *scale_plane; int idx_bits, main_bits, aux_bits, qmax;
};

// ORs `width` bits of `val` into a little-endian bit stream at bit `pos` of `row` (the field holds zeros); other
// threads may do the same to neighbouring fields of the same bytes.
__device__ __forceinline__ void or_bit_field(uint8_t *row, int pos, uint32_t val, int width) {
    if (width <= 0 || val == 0u) return;
    const uint64_t v = (uint64_t)(val & ((1u << width) - 1u)) << (pos & 7);
    uint8_t *p = row + (pos >> 3);
    for (int i = 0; i * 8 < (pos & 7) + width; i++) {
        const uint32_t byte = (uint32_t)(v >> (8 * i)) & 0xffu;
        if (!byte) continue;
        const uintptr_t a = (uintptr_t)(p + i);
        atomicOr(reinterpret_cast<uint32_t *>(a & ~(uintptr_t)3), byte << (8 * (a & 3)));
    }
}

// A flagged chunk for which the sideband has no room left degrades to a plain HQMQ chunk: its flag bit is cleared and
// the radius code that the quantizer would have stored for an unflagged chunk is written into its (zero) radius field
// (the reference never loses an outlier, src/quantizers/outlier_aware.py:86; a full sideband costs accuracy here, not
// the chunk).  xc: the chunk's four input values; prow: the row's index in the [B][H][t_cap] planes.
// Built with -ffp-contract=off like the quantizer: the same roundings, the same code.
template <class D>
__device__ __forceinline__ void degrade_to_plain(const CompactCall &a, size_t prow, int c, const typename D::storage *xc) {
    if (!a.main_plane || !a.scale_plane) return;
    const float nrm = D::rnd(norm4(D::load(xc), D::load(xc + 1), D::load(xc + 2), D::load(xc + 3)));
    const float r = clamp_min_d<D>(nrm, 1e-8f);
    const float rm = D::load((const typename D::storage *)a.scale_plane + prow);
    const float qmaxf = (float)a.qmax;
    const float scale = D::rnd(rm / qmaxf);
    float qf = rintf(D::rnd(r / scale));
    if (!is_nan(qf)) qf = fminf(fmaxf(qf, 0.f), qmaxf);
    const uint32_t rq = is_nan(qf) ? 0u : (uint32_t)(int)qf;
    const int in_main = a.main_bits - a.idx_bits;                  // radius bits that live in the main field
    if (in_main > 0) or_bit_field(a.main_plane + prow * (size_t)((a.n * a.main_bits + 7) >> 3), c * a.main_bits + a.idx_bits, rq, in_main);
    if (a.aux_plane && a.aux_bits > 0)
        or_bit_field(a.aux_plane + prow * (size_t)((a.n * a.aux_bits + 7) >> 3), c * a.aux_bits, in_main > 0 ? rq >> in_main : rq, a.aux_bits);
    const uintptr_t fa = (uintptr_t)(const_cast<uint8_t *>(a.flag_plane) + prow * (size_t)((a.n + 7) >> 3) + (c >> 3));
    atomicAnd(reinterpret_cast<uint32_t *>(fa & ~(uintptr_t)3), ~((1u << (c & 7)) << (8 * (fa & 3))));
}
int med3x_calls(const Med3xCall *c, int count, hipStream_t st);                                            // med3x.hip
int compact_calls(const CompactCall *c, int count, hipStream_t st);                                        // med3x.hip
int check_compact(const CompactCall &c);                                                                   // med3x.hip
// ck / cv (may be NULL): the compaction that follows; compacted[i] tells whether the quantize launch did it
int quantize_two(const hqmq_quantize_args *k, const hqmq_quantize_args *v, const CompactCall *ck, const CompactCall *cv,
                 bool compacted[2], hipStream_t st);                                                           // quantize.hip

}  // namespace hqmq
