// Types and device helpers shared by the generic and the specialised attention kernels.
#pragma once
#include "common.h"
#include <hip/hip_ext.h>

namespace hqmq {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kAttnWaves = 4;
constexpr int kSuper = 64;  // tokens per super-tile
constexpr int kPartialHead = 4;  // floats in front of the accumulators of a split partial (m, l, 2 unused): keeps acc 16-byte aligned

struct PackedDev {
    const uint8_t *main_plane, *aux_plane, *flag_plane;
    const void *scale_plane;
    int64_t ssb, ssh, sst;
    const void *sideband;
    const int32_t *sb_tile_off;
    int64_t sb_cap;
    const uint16_t *sb_coord;
    const int32_t *sb_count;
    const void *joint;
    int64_t jsh;
    int K;
    const uint32_t *scale_max;
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
    const int32_t *kv_start;   // [B] or NULL: the first visible token of every sequence (left padding)
    const int32_t *batch_order; // [B] or NULL: a permutation of the sequences, the order their blocks start in
    int causal;
    int64_t causal_offset;
    float c_log2;   // softmax_scale * log2(e) / qmax
    float c_plain;  // softmax_scale * log2(e)
    float inv_qmax;
    int n_splits, n_cg;
    int scale_vec;  // scales of 4 consecutive tokens may be read with one aligned vector load
    float *ws;      // split partials [row][split][kPartialHead + d_h]: m (base-2 exponent units), l, two unused floats, acc
    int xcd_remap;  // blocks of one (sequence, KV head) share an XCD (see attn_fast_kernel)
    // multipliers that replace the index divisions of the kernels' prologue (attn_div_magic; 0 = divide)
    unsigned m_hkv, m_G, m_gz, m_gx, m_splits;
    int tab_fp8;    // both tables hold e4m3 numbers and the caller asks for float8 storage in LDS
    int wide_range; // scales or verbatim values of the cache may leave the fp16 range: layout-generic kernel only
    int no_lds_landing; // keep the specialised kernels that hold their tiles in registers (testing, measurements)
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
    // tiles never written (or cropped) hold INT32_MAX: bound the offset before adding to it
    const int tile_off = min(c.sb_tile_off[tile_off_index], (int)min(c.sb_cap, (int64_t)0x3fffffff));
    slot0 = max(tile_off, 0) + pre_t + __popc(fw_t & ((first >= 32) ? 0xffffffffu : ((1u << first) - 1u)));
}

// A flagged chunk: the verbatim values from the sideband (exact in fp16 for fp16 caches), times `down`: 1, or the
// power of two that brings a bf16 / fp32 cache whose values leave the fp16 range back into it (a verbatim value is
// bounded by its token's scale, so the bound of the scales serves).
__device__ __forceinline__ half4 outlier_chunk(const PackedDev &c, int dtype, size_t bh, int slot, float down) {
    int64_t s = slot;
    if (s >= c.sb_cap) s = c.sb_cap - 1;
    if (s < 0) s = 0;
    const int64_t chunk = (int64_t)bh * c.sb_cap + s;
    if (dtype == HQMQ_F16) return load_chunk_h(c.sideband, dtype, chunk);
    half4 r;
    for (int j = 0; j < 4; j++) r[j] = (_Float16)(load_any(c.sideband, dtype, chunk * 4 + j) * down);
    return r;
}


// Copies one head's joint table (K rows of 4 elements in `dtype`) into LDS as fp16. Loads are issued in
// batches so that their latencies overlap instead of adding up.
__device__ __forceinline__ void fill_table(uint2 *dst, const void *joint, int dtype, int64_t first_chunk, int K) {
    constexpr int U = 6;
    const int step = blockDim.x;
    for (int k0 = threadIdx.x; k0 < K; k0 += step * U) {
        half4 tmp[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * step;
            tmp[u] = k < K ? load_chunk_h(joint, dtype, first_chunk + k) : half4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + u * step;
            if (k < K) dst[k] = __builtin_bit_cast(uint2, tmp[u]);
        }
    }
}

// ceil(2^32 / d) if x / d == umulhi(x, that) for every x <= x_max (true while x_max * d < 2^32), else 0
inline unsigned attn_div_magic(uint64_t d, uint64_t x_max) {
    if (d < 2 || x_max * d >= (1ull << 32)) return 0u;
    return (unsigned)(((1ull << 32) + d - 1) / d);
}

// Power-of-two offset of the softmax exponent that keeps P * (V scale) inside fp16's normal range: 0 while the
// largest V scale lies in [2^-8, 2^15); above, its excess exponent; below (a cache of tiny values, whose products
// would be fp16 subnormals), the negative exponent that brings the largest scale to [0.5, 1).  Numerator and
// denominator of the attention output carry the same factor.
__device__ __forceinline__ int v_scale_shift_bits(const PackedDev &v) {
    if (!v.scale_max) return 0;
    const uint32_t bits = __builtin_amdgcn_readfirstlane(__builtin_nontemporal_load(v.scale_max));      // wave-uniform
    if (bits == 0u) return 0;                                   // nothing written yet
    const int e = (int)((bits >> 23) & 0xffu) - 127 + 1;        // scale < 2^e
    return e > 15 ? e - 15 : e < -8 ? max(e, -64) : 0;        // at most 2^64 upwards: the fp32 sum of the weights stays finite
}
__device__ __forceinline__ float v_scale_shift(const PackedDev &v) { return (float)v_scale_shift_bits(v); }

// Implemented in attention_fast.hip: kernels specialised at compile time for the common layouts
// (d_h 64/128, fp16/bf16 caches; 16+0 / 12+1 / 16+3 bit codes, and at d_h 128 the widths 16+1, 16+2, 12+2, 12+3). Returns HQMQ_OK and sets *handled when
// it launched one of them; otherwise the caller falls back to the generic kernel.
// Optional events that receive the GPU timestamps of the begin and the end of the main attention kernel.
struct LaunchTiming {
    hipEvent_t start = nullptr, stop = nullptr;
};
template <class Kern>
inline void launch_timed(Kern kern, dim3 grid, dim3 block, size_t shmem, hipStream_t st, const LaunchTiming &tm, const AttnParams &p) {
    if (tm.start || tm.stop) hipExtLaunchKernelGGL(kern, grid, block, shmem, st, tm.start, tm.stop, 0, p);
    else hipLaunchKernelGGL(kern, grid, block, shmem, st, p);
}

int launch_attn_fast(const AttnParams &p, int main_bits, bool flags, dim3 grid, size_t table_bytes, hipStream_t st,
                     const LaunchTiming &tm, bool *handled);

}  // namespace hqmq
