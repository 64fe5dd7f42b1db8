// Attention kernels specialised at compile time for the layouts of the benchmark shapes:
// d_h = 64 / 128, fp16 or bf16 caches, codes of 16+0 (s96_r4), 12+1 (s24_r3) or 16+3 (s192_r6) bits.
//
// Lane mapping (one wavefront, one 16-token tile): lane = 16 * grp + col decodes the CPL = d_h / 16 chunks
// grp * CPL ... of token `col`, for K and for V alike.
//   S^T = K . Q^T     v_mfma_f32_16x16x32_f16: A = two decoded K chunks of the lane, B = the matching Q chunks.
//   V^T               the A operand of O^T = V^T . P^T needs 4 tokens of one d per lane, a decoded chunk is
//                     4 d of one token.  The 16x16 transposition is one v_mfma_f32_16x16x16_f16 against the
//                     identity (exact: every output is one fp16 input times 1.0) and two packed conversions,
//                     instead of a dozen cross-lane VALU operations per chunk.
//   O^T += V^T . P^T  v_mfma_f32_16x16x32_f16 over two tiles (32 tokens) at a time.
// Row j of the V-side product is d = (grp * CPL + j) * 4 + e, the order the epilogue writes back.
// Scores are kept as S^T * rs; 1/qmax is folded into the softmax scale and the epilogue.  Outlier chunks
// carry radius code 0 in the planes, so they decode to zero; their verbatim values enter through extra MFMAs
// that walk the sideband entry list (values + coordinates), never the flag plane.
#include "attention_common.h"
#include <cstdlib>

namespace hqmq {

// Time stamps inside the kernels: measurement builds only (-DHQMQ_STAMPS, libhqmq_amd_stamps.so)
#ifdef HQMQ_STAMPS
__device__ unsigned long long *g_stamps;
#define STAMP(i) do { st_[i] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define STAMP(i) do { } while (0)
#endif
#if defined(HQMQ_STAMPS) && HQMQ_STAMPS + 0 >= 2     // -DHQMQ_STAMPS=2: time per phase of the outlier variants' half-steps (the stamps cost time themselves)
#define PHASE(i) do { if constexpr (FLAGS) { const unsigned long long t_ = __builtin_amdgcn_s_memrealtime(); ph_[i] += t_ - tl_; tl_ = t_; } } while (0)
#else
#define PHASE(i) do { } while (0)
#endif

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef const uint2 __attribute__((address_space(3))) *lds_u2_ptr;
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint4v uint4v_a8 __attribute__((aligned(8)));         // a 16-byte vector at an 8-byte aligned address
typedef uint32_t uint32_a2 __attribute__((aligned(2)));       // a dword at a 2-byte aligned address

template <int DT>
__device__ __forceinline__ half4 chunk_to_half(uint2 w) {
    if (DT == HQMQ_F16) return __builtin_bit_cast(half4, w);
    half4 r;
    r[0] = (_Float16)__uint_as_float(w.x << 16); r[1] = (_Float16)__uint_as_float(w.x & 0xffff0000u);
    r[2] = (_Float16)__uint_as_float(w.y << 16); r[3] = (_Float16)__uint_as_float(w.y & 0xffff0000u);
    return r;
}

// Two codewords (16 bytes) of a table in the cache dtype -> the same two as fp16
template <int DT>
__device__ __forceinline__ uint4v pair_to_half(uint4v w) {
    if (DT == HQMQ_F16) return w;
    const uint2 a = __builtin_bit_cast(uint2, chunk_to_half<DT>(uint2{w[0], w[1]}));
    const uint2 b = __builtin_bit_cast(uint2, chunk_to_half<DT>(uint2{w[2], w[3]}));
    return uint4v{a.x, a.y, b.x, b.y};
}

// One codeword (four fp16 in two dwords) of e4m3 numbers -> four float8 bytes (exact)
__device__ __forceinline__ uint32_t codeword_to_f8(uint32_t w0, uint32_t w1) {
    const half2v a = __builtin_bit_cast(half2v, w0), b = __builtin_bit_cast(half2v, w1);
    int v = __builtin_amdgcn_cvt_pk_fp8_f32((float)a[0], (float)a[1], 0, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32((float)b[0], (float)b[1], v, true);
    return (uint32_t)v;
}
// Two codewords of a table whose entries are e4m3 numbers -> the same two as eight float8 bytes
template <int DT>
__device__ __forceinline__ uint2 pair_to_f8(uint4v w) {
    const uint4v h = pair_to_half<DT>(w);
    const uint32_t h0 = h[0], h1 = h[1], h2 = h[2], h3 = h[3];
    return uint2{codeword_to_f8(h0, h1), codeword_to_f8(h2, h3)};
}
template <int DT, bool F8>
__device__ __forceinline__ void store_pair(void *tab, int k, uint4v w) {
    if constexpr (F8) reinterpret_cast<uint2 *>(tab)[k] = pair_to_f8<DT>(w);
    else reinterpret_cast<uint4v *>(tab)[k] = pair_to_half<DT>(w);
}

// The parameter block spans several 64-byte lines of the kernel-argument segment, and the prologue reads them one
// after the other as its address arithmetic proceeds: every first touch of a line is a miss of the scalar cache
// that the next scalar load waits behind.  One dword of every line, requested together at the very start, turns
// the chain of misses into one.
__device__ __forceinline__ void touch_kernargs() {
    typedef const uint32_t __attribute__((address_space(4))) *karg_ptr;
    karg_ptr ka = (karg_ptr)__builtin_amdgcn_kernarg_segment_ptr();
    uint32_t t = 0;
#pragma unroll
    for (int i = 0; i < (int)((sizeof(AttnParams) + 63) / 64); i++) t |= ka[16 * i];
    asm volatile("" ::"s"(t));
}

// One word of a caller's array that no kernel writes while this one runs, at a wave-uniform index: read through the
// constant address space, i.e. by a scalar load.  (As a vector load it is followed by a wait for every vector load
// before it: in the prologues below, for the table loads, and once per dependent word.)
__device__ __forceinline__ int32_t uniform_word(const int32_t *a, int64_t i) {
    typedef const int32_t __attribute__((address_space(4))) *const_i32_ptr;
    return ((const_i32_ptr)(uintptr_t)a)[i];
}

constexpr int kFastWaves = 8;     // wavefronts per block; 12 (three per SIMD) for plain 16+0 caches with long ranges per block

// codes, aux bits and raw 16-bit scales of 32 tokens (two 16-token tiles) for one lane
template <int NW, int AB, bool FLAGS>
struct HalfTile {
    uint32_t kw[2][NW], vw[2][NW];
    uint32_t kaux[AB ? 2 : 1], vaux[AB ? 2 : 1];
    uint2 ks[2], vs[2];
};
// outlier bookkeeping of the same 32 tokens; it travels one half-step ahead of the codes, so that the sideband
// chunks it points to can be requested a whole half-step before use
struct FlagTile {
    int koff[3];               // K: sideband entries [koff[u], koff[u + 1]) belong to tile u (wave-uniform)
    int voff[3];               // V: the same
};
// K outliers of one half-step, requested ahead: the first NB batches of eight sideband entries.  Lane
// 16 * grp + col holds entries 2 * grp and 2 * grp + 1 of a batch (the same in all 16 lanes of a row).
template <int NB>
struct KPre {
    int off[3];
    uint4v x[NB];              // two verbatim chunks (raw bits of the cache dtype) as loaded, see k_load
    uint32_t cc[NB];           // their coordinates as loaded: (token & 15) << 8 | chunk, two 16-bit fields
};
// V outliers of one half-step: the first NB batches of sixteen entries; lane 16 * grp + col holds entry `col`.
template <int NB>
struct VPre {
    int off[3];
    uint2 x[NB];
    uint32_t cc[NB];
};
// the unit of prefetch: NH half-tiles of 32 tokens
template <int NW, int AB, bool FLAGS, int NH>
struct FastTile {
    HalfTile<NW, AB, FLAGS> h[NH];
};

template <int NBYTES>
__device__ __forceinline__ uint32_t load_small(const uint8_t *p) {
    if constexpr (NBYTES == 4) return *reinterpret_cast<const uint32_t *>(p);
    else if constexpr (NBYTES == 2) return *reinterpret_cast<const uint16_t *>(p);
    else {
        uint32_t v = 0;
#pragma unroll
        for (int i = 0; i < NBYTES; i++) v |= (uint32_t)p[i] << (8 * i);
        return v;
    }
}

// two 16-bit scales (raw bits of dtype DT) as a packed fp16 pair
template <int DT>
__device__ __forceinline__ half2v scale_h2(uint32_t pair) {
    if (DT == HQMQ_F16) return __builtin_bit_cast(half2v, pair);
    half2v r;
    r[0] = (_Float16)__uint_as_float(pair << 16);
    r[1] = (_Float16)__uint_as_float(pair & 0xffff0000u);
    return r;
}
// acc * scale[hi] (+ add): for fp16 scales one mixed-precision fma reads the half directly
template <int DT>
__device__ __forceinline__ float scaled(float acc, uint32_t pair, int hi, float add) {
    if (DT == HQMQ_F16) return __builtin_fmaf(acc, (float)__builtin_bit_cast(half2v, pair)[hi], add);
    return __builtin_fmaf(acc, __uint_as_float(hi ? (pair & 0xffff0000u) : (pair << 16)), add);
}

// The dynamic LDS block is the kernel's only LDS, so it starts at LDS address 0: the K table sits at byte 0,
// the V table at kVTabOffset, and a gather addresses them with idx * 8 (+ the instruction's immediate offset).
constexpr int kVTabOffset = 40960;          // bytes; room for 5120 K codewords in front of it
constexpr int kQOffset = kVTabOffset + 36864;     // outlier variants: Q as [chunk][column] fp16 chunks, after the V table
constexpr int kFlagsTabMax = (kQOffset - kVTabOffset) / 8;      // codewords the V slot of the outlier variants holds
static_assert(kFlagsTabMax * 8 + kVTabOffset == kQOffset && kFlagsTabMax == 4608, "V table slot of the outlier variants");
constexpr int kAuxTabOffset = 36864;        // s192_r6: 64 dwords with the high radius bits of a pair of chunks, see gather_chunks
// s24_r3 (13-bit codes, K <= 1024, qmax = 7): the tables are kept multiplied out, entry [rq][idx] = codeword * rq at byte
// (rq << 10 | idx) * 8, so that the 13-bit code is the table index and a decode is one gather (no radius arithmetic).
constexpr int kPsTabBytes = 8 * 1024 * 8;   // 64 KB per tensor
constexpr bool is_prescaled(int CPL, int MB, int AB, int IB) { return CPL == 8 && MB == 12 && AB == 1 && IB == 10; }
constexpr int vtab_offset(bool ps) { return ps ? kPsTabBytes : kVTabOffset; }
constexpr int q_offset(bool ps) { return ps ? 2 * kPsTabBytes : kQOffset; }
constexpr int sel_offset(bool ps) { return q_offset(ps) + 4096; }      // nine rows of eight fp16: row r < 8 = qmax times unit vector r, row 8 = 0
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef const uint4v __attribute__((address_space(3))) *lds_u4_ptr;
typedef const uint32_t __attribute__((address_space(3))) *lds_u1_ptr;

template <int TAB_OFF>
__device__ __forceinline__ half4 gather8(uint32_t byte_addr) {
    return __builtin_bit_cast(half4, *(lds_u2_ptr)(uintptr_t)(byte_addr + TAB_OFF));
}

// Table byte address of the low (HI = 0) or high (HI = 1) 16-bit index of a masked pair: one shift that reads
// a half of the register (the compiler's own lowering is a shift and an and).
template <int HI>
__device__ __forceinline__ uint32_t half_addr8(uint32_t pair) {
    uint32_t r;
    if constexpr (HI)
        asm("v_lshlrev_b32_sdwa %0, 3, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1" : "=v"(r) : "v"(pair));
    else
        asm("v_lshlrev_b32_sdwa %0, 3, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_0" : "=v"(r) : "v"(pair));
    return r;
}

// The same for a table kept as float8 e4m3 (F8 variants: four bytes per codeword, for tables whose entries are e4m3
// numbers): one 32-bit LDS read and two conversions that widen two bytes each to packed fp16 (exact).
template <int TAB_OFF>
__device__ __forceinline__ half4 gather4_f8(uint32_t byte_addr) {
    const uint32_t w = *(lds_u1_ptr)(uintptr_t)(byte_addr + TAB_OFF);
    const half2v lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
    const half2v hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
    return half4{lo[0], lo[1], hi[0], hi[1]};
}
template <int HI>
__device__ __forceinline__ uint32_t half_addr4(uint32_t pair) {
    uint32_t r;
    if constexpr (HI)
        asm("v_lshlrev_b32_sdwa %0, 2, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1" : "=v"(r) : "v"(pair));
    else
        asm("v_lshlrev_b32_sdwa %0, 2, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_0" : "=v"(r) : "v"(pair));
    return r;
}
template <int TAB_OFF, bool F8, int HI>
__device__ __forceinline__ half4 gather_pair_half(uint32_t ix) {
    if constexpr (F8) return gather4_f8<TAB_OFF>(half_addr4<HI>(ix));
    else return gather8<TAB_OFF>(half_addr8<HI>(ix));
}

// Decode of the CPL chunks of one lane in two steps, so that a caller can put all gathers of a half-step in flight
// before the first multiply: gather_chunks requests the codewords from the LDS table (g) and prepares the radius
// codes as packed fp16 pairs (r, chunk j in r[j / 2][j & 1]); scale_chunks multiplies.
// 16+0 layout: the two radius codes of a dword become an fp16 pair with one shift, one and-or
// (0x6400 | rq is the fp16 number 1024 + rq) and one packed subtract.  IB = idx_bits when known at compile
// time (12 for s96), else 0.
template <int CPL, int MB, int AB, int IB, int NW, int TAB_OFF, bool F8 = false>
__device__ __forceinline__ void gather_chunks(const uint32_t (&w)[NW], uint32_t aux, int idx_bits_rt, half4 (&g)[CPL], half2v (&r)[CPL / 2]) {
    const int idx_bits = IB ? IB : idx_bits_rt;
    const uint32_t idx_mask = (1u << idx_bits) - 1u;
    const half2v k1024 = half2v{(_Float16)1024.0f, (_Float16)1024.0f};
    if constexpr (MB == 16 && AB == 0) {
        // mask in a scalar register and magic in a vector register, so that (x & mask) | magic is one v_and_or_b32
        uint32_t rq2 = (0xffffu >> idx_bits) * 0x00010001u, magic = 0x64006400u;
        asm("" : "+s"(rq2));
        asm("" : "+v"(magic));
        const uint32_t im2 = idx_mask * 0x00010001u;
#pragma unroll
        for (int i = 0; i < CPL / 2; i++) {
            const uint32_t ix = w[i] & im2;
            g[2 * i] = gather_pair_half<TAB_OFF, F8, 0>(ix);
            g[2 * i + 1] = gather_pair_half<TAB_OFF, F8, 1>(ix);
            const uint32_t t = ((w[i] >> idx_bits) & rq2) | magic;
            r[i] = __builtin_bit_cast(half2v, t) - k1024;
        }
    } else if constexpr (MB == 16 && AB == 3 && IB == 13) {
        // s192_r6: idx (13 bits) and the low three radius bits in the 16-bit main field, the high three in the aux
        // row.  Six aux bits (two chunks) index a 64-entry LDS table holding them at bits 3..5 and 19..21 together
        // with the 0x6400 fp16 magic.
        constexpr uint32_t im2 = 0x1fff1fffu;
#pragma unroll
        for (int i = 0; i < CPL / 2; i++) {
            const uint32_t ix = w[i] & im2;
            g[2 * i] = gather_pair_half<TAB_OFF, F8, 0>(ix);
            g[2 * i + 1] = gather_pair_half<TAB_OFF, F8, 1>(ix);
            const uint32_t hi = *(lds_u1_ptr)(uintptr_t)(kAuxTabOffset + ((aux >> (6 * i)) & 63u) * 4u);
            const uint32_t t = ((w[i] >> 13) & 0x00070007u) | hi;
            r[i] = __builtin_bit_cast(half2v, t) - k1024;
        }
    } else if constexpr (MB == 12 && AB == 1 && IB == 10 && CPL == 8) {
        static_assert(!F8, "the float8 table variants exist for 16-bit main fields");
        // s24_r3, tables multiplied out (see kPsTabBytes): eight 12-bit fields (idx in the low 10 bits, the low two
        // radius bits above) in three dwords and one aux byte with the eight high radius bits; field | aux bit << 12 is
        // the table index.  No radius arithmetic: r stays unused.
        const uint32_t w0 = w[0], w1 = w[1], w2 = w[2];
        constexpr uint32_t M = 0x7ff8u;
        const uint32_t ad[8] = {(w0 << 3) & M, (w0 >> 9) & M, __builtin_amdgcn_alignbit(w1, w0, 21) & M, (w1 >> 1) & M,
                                (w1 >> 13) & M, __builtin_amdgcn_alignbit(w2, w1, 25) & M, (w2 >> 5) & M, (w2 >> 17) & M};
#pragma unroll
        for (int j = 0; j < 8; j++) g[j] = gather8<TAB_OFF>(((aux << (15 - j)) & 0x8000u) | ad[j]);
    } else {
        static_assert(!F8, "the float8 table variants exist for the layouts with compile-time index widths");
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            uint32_t code = code_at<MB, NW>(w, j);
            if (AB) code |= ((aux >> (j * AB)) & ((1u << AB) - 1u)) << MB;
            g[j] = gather8<TAB_OFF>((code & idx_mask) << 3);
            r[j >> 1][j & 1] = (_Float16)(uint16_t)(code >> idx_bits);
        }
    }
}
template <int CPL, bool PS = false>
__device__ __forceinline__ void scale_chunks(const half4 (&g)[CPL], const half2v (&r)[CPL / 2], half4 (&a)[CPL]) {
#pragma unroll
    for (int j = 0; j < CPL; j++) a[j] = PS ? g[j] : g[j] * r[j >> 1][j & 1];
}

// x / d through the multiplier the host worked out for d (m = ceil(2^32 / d), exact while x * d < 2^32; m = 0 stands for
// d = 1: the launcher keeps these kernels for launches where every divisor has its multiplier, see launch_layout).
// No division as a fall-back: its expansion, once per use, made the prologue a chain of branches, each with its own
// re-read of the argument block and a wait for it.
__device__ __forceinline__ unsigned fast_div(unsigned x, unsigned d, unsigned m) { return m ? __umulhi(x, m) : x; }

__device__ __forceinline__ half8 cat8(half4 x, half4 y) { return __builtin_shufflevector(x, y, 0, 1, 2, 3, 4, 5, 6, 7); }

// max over the four 16-lane rows (lanes l, l^16, l^32, l^48) without going through LDS
__device__ __forceinline__ float row_max4(float x) {
    const uint32_t b = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const float y = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    const uint32_t c = __float_as_uint(y);
    const auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
    return fmaxf(__uint_as_float(q[0]), __uint_as_float(q[1]));
}
__device__ __forceinline__ float row_sum4(float x) {
    const uint32_t b = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const float y = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    const uint32_t c = __float_as_uint(y);
    const auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

// fp32 4-vector (exact fp16 values) -> packed fp16
__device__ __forceinline__ half4 pack4(float4v t) {
    const auto lo = __builtin_amdgcn_cvt_pkrtz(t[0], t[1]);
    const auto hi = __builtin_amdgcn_cvt_pkrtz(t[2], t[3]);
    return __builtin_bit_cast(half4, uint2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)});
}

// NCG: column groups (of 16 columns) per wavefront.  Two for chunked prefill with more than 16 columns per KV head:
// a decoded tile and its V transposition then serve 32 columns.
// F8: the codeword tables are kept as float8 e4m3 in LDS (callers that rounded their tables to e4m3)
template <int CPL, int MB, int AB, int IB, int DT, bool FLAGS, int WV = kFastWaves, int NCG = 1, bool F8 = false>
__global__ __launch_bounds__(WV * 64, WV == 12 ? 3 : 2) void attn_fast_kernel(AttnParams p) {
    static_assert(NCG == 1 || !FLAGS, "outlier variants take one column group");
    constexpr int NB = CPL * MB / 8;
    constexpr int NW = (NB + 3) / 4;
    constexpr int ABYTES = CPL * AB / 8;     // aux bytes per lane (CPL * AB is a multiple of 8 here)
    static_assert(AB == 0 || (CPL * AB) % 8 == 0, "aux bits of one lane must be whole bytes");
    static_assert(CPL % 2 == 0, "two chunks per 16x16x32 operand");
    constexpr int NT = WV * 64;
    constexpr int kKPre = CPL >= 8 ? 3 : 1;     // batches of outlier entries requested ahead (d_h 64 has half the chunks)
    constexpr bool kBatchGathers = false;       // see half_step: measured, no gain on any shape (178 against 157 registers)
    constexpr int NH = 1;       // half-steps per prefetched tile: one measures faster than two on every shape
    extern __shared__ uint2 lds_tab[];
#ifdef HQMQ_STAMPS
    unsigned long long ph_[8] = {}, tl_ = 0;         // outlier variants: time per phase of the half-steps, summed per wavefront
    int n_steps_ = 0;
    const unsigned long long t_in_ = __builtin_amdgcn_s_memrealtime();
    unsigned long long t_loop_ = 0;
#endif
    constexpr bool PS = is_prescaled(CPL, MB, AB, IB);
    constexpr int VTAB = vtab_offset(PS), QOFF = q_offset(PS), SELOFF = sel_offset(PS);
    uint2 *ktab = lds_tab, *vtab = lds_tab + VTAB / 8;
    touch_kernargs();

    // blocks are dispatched in grid order: batch_order lists the sequences in the order they should start
    // (longest first for ragged batches, so that no long sequence is left for the end)
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    if (p.xcd_remap) {
        // the hardware hands workgroups to the XCDs round-robin in linear order (x fastest): renumber so that the
        // (sequence, KV head) index runs fastest and, with a multiple of eight of them, stays on one XCD
        const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const unsigned r = fast_div(lin, gridDim.z, p.m_gz);
        bz = (int)(lin - r * gridDim.z);
        by = (int)fast_div(r, gridDim.x, p.m_gx);
        bx = (int)(r - (unsigned)by * gridDim.x);
    }
    const int slot = (int)fast_div((unsigned)bz, (unsigned)p.Hkv, p.m_hkv);
    // Consecutive sequences start with different KV heads: with eight heads (or a multiple) block index modulo 8, and
    // so the XCD, would otherwise always be the same head, and heads differ in cost (config 4: 20 to 45 sideband
    // entries per half-step and head, 2.8 to 3.4 us per half-step: the XCD of the densest head finished 20 % after
    // the others).
    // (With fewer than eight heads, 8 / Hkv consecutive sequences fill one round of the XCDs and share a rotation.)
    const int turn = slot >> (p.Hkv == 4 ? 1 : p.Hkv == 2 ? 2 : p.Hkv == 1 ? 3 : 0);
    int hkv = bz - slot * p.Hkv + (turn - (int)fast_div((unsigned)turn, (unsigned)p.Hkv, p.m_hkv) * p.Hkv);
    if (hkv >= p.Hkv) hkv -= p.Hkv;
    // The codeword-table loads are the longest dependency chain of the prologue (load, convert, LDS store, barrier)
    // and need nothing but the KV head: they are requested before anything else is worked out.  16-byte loads of two
    // codewords, all unconditional (clamped): straight-line code, exact wait counts.
    // (every pair of the largest table the LDS slots hold, 2560 pairs, in one round of requests: a second round would
    // be a loop of loads, and the wait at its head covers every request in flight, the first tile's included)
    constexpr int FU = is_prescaled(CPL, MB, AB, IB) ? (512 + NT - 1) / NT : (kVTabOffset / 16 + NT - 1) / NT;
    const uint4v *ksrc = (const uint4v *)((const uint2 *)p.Kc.joint + hkv * (p.Kc.jsh / 4));
    const uint4v *vsrc = (const uint4v *)((const uint2 *)p.Vc.joint + hkv * (p.Vc.jsh / 4));
    const int Kk2 = p.Kc.K >> 1, Kv2 = p.Vc.K >> 1;        // tables of an even number of codewords (checked at launch)
    uint4v tk[FU], tv[FU];
#pragma unroll
    for (int u = 0; u < FU; u++) {
        const int k = threadIdx.x + u * NT;
        tk[u] = ksrc[min(k, Kk2 - 1)];
        tv[u] = vsrc[min(k, Kv2 - 1)];
    }
#ifdef HQMQ_STAMPS
    ph_[0] = __builtin_amdgcn_s_memrealtime();      // table loads requested
#endif
    const int b = p.batch_order ? min(max(uniform_word(p.batch_order, slot), 0), p.B - 1) : slot;
    const int bh = b * p.Hkv + hkv;
    const int cg0 = by * NCG, sp = bx;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int G = p.G;
    constexpr int n = 4 * CPL, d_h = 16 * CPL;
    const int col = lane & 15, grp = lane >> 4;
    // The four per-sequence words go out together, without a branch on the optional pointers (an absent array reads
    // a word of the kernel arguments instead): one scalar round trip instead of one per word.
    const int32_t *const spare_word = (const int32_t *)(uintptr_t)__builtin_amdgcn_kernarg_segment_ptr();
    const int32_t w_len = uniform_word(p.kv_len ? p.kv_len + b : spare_word, 0);
    const int32_t w_start = uniform_word(p.kv_start ? p.kv_start + b : spare_word, 0);
    const int32_t w_kcount = uniform_word(FLAGS ? p.Kc.sb_count + bh : spare_word, 0);
    const int32_t w_vcount = uniform_word(FLAGS ? p.Vc.sb_count + bh : spare_word, 0);
    int kv_end = p.kv_len ? w_len : p.Tkv;
    kv_end = min(max(kv_end, 0), p.Tkv);
    bool col_ok[NCG];
    int tq[NCG], hq[NCG], col_lim[NCG];
    int blk_lim = 0, lim_min = 0x7fffffff;
#pragma unroll
    for (int cgi = 0; cgi < NCG; cgi++) {
        const int cidx = (cg0 + cgi) * 16 + col;
        col_ok[cgi] = cidx < p.Tq * G;
        tq[cgi] = col_ok[cgi] ? (int)fast_div((unsigned)cidx, (unsigned)G, p.m_G) : 0;
        hq[cgi] = hkv * G + (col_ok[cgi] ? cidx - tq[cgi] * G : 0);
        int64_t lim64 = kv_end;
        if (p.causal) lim64 = min(lim64, (int64_t)tq[cgi] + p.causal_offset + 1);
        if (!col_ok[cgi] || lim64 < 0) lim64 = 0;
        col_lim[cgi] = (int)lim64;
        blk_lim = max(blk_lim, col_lim[cgi]);
        if (col_ok[cgi]) lim_min = min(lim_min, col_lim[cgi]);
    }
    if (p.causal) {
        for (int o = 1; o < 16; o <<= 1) {
            blk_lim = max(blk_lim, __shfl_xor(blk_lim, o));
            lim_min = min(lim_min, __shfl_xor(lim_min, o));
        }
        blk_lim = __builtin_amdgcn_readfirstlane(blk_lim);      // the same in every lane: all rows hold all 16 columns
        lim_min = __builtin_amdgcn_readfirstlane(lim_min);
    } else {
        blk_lim = lim_min = kv_end;         // every column in range sees the whole sequence (a launched block has one)
    }
    // tokens before kv_start[b] are invisible (left padding): the walk starts at the super-tile that holds it
    const int col_start = p.kv_start ? min(max(w_start, 0), blk_lim) : 0;
    const int blk_lo = col_start / kSuper * kSuper;
    int per_split = (int)fast_div((unsigned)(blk_lim - blk_lo + p.n_splits - 1), (unsigned)p.n_splits, p.m_splits);
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int b_begin = min(blk_lo + sp * per_split, blk_lim), b_end = min(blk_lim, b_begin + per_split);
    // The block's half-steps go to its wavefronts round-robin: wavefront w takes the 32 tokens at b_begin + 32 (w + i WV),
    // i = 0, 1, ...  What the wavefronts of a block request at any one time is then one contiguous stretch of the
    // planes (batch 8: 3.5 % faster than a contiguous range per wavefront, ragged config 4: 2 %).
    // Every half-step starts at a multiple of 32 below T_kv <= t_cap (a multiple of 64): whole tiles are readable.
    constexpr int TS = 32 * WV;
    const int t_begin = min(b_begin + wave * 32, b_end), t_end = b_end;
    const size_t plane_row0 = (size_t)bh * p.t_cap;
    constexpr int mrb = n * MB / 8, arb = (n * AB + 7) / 8;
    const int64_t tiles_cap = p.t_cap / kTile;
    const int tiles_cap1 = (int)tiles_cap - 1;
    const int idx_bits = p.idx_bits;
    const uint16_t *ks_plane = (const uint16_t *)p.Kc.scale_plane + b * p.Kc.ssb + hkv * p.Kc.ssh;
    const uint16_t *vs_plane = (const uint16_t *)p.Vc.scale_plane + b * p.Vc.ssb + hkv * p.Vc.ssh;
    const uint8_t *k_rows = p.Kc.main_plane + plane_row0 * mrb;
    const uint8_t *v_rows = p.Vc.main_plane + plane_row0 * mrb;
    const uint8_t *ka_rows = AB ? p.Kc.aux_plane + plane_row0 * arb : nullptr;
    const uint8_t *va_rows = AB ? p.Vc.aux_plane + plane_row0 * arb : nullptr;
    const int32_t *k_toff = FLAGS ? p.Kc.sb_tile_off + (size_t)bh * tiles_cap : nullptr;
    const int32_t *v_toff = FLAGS ? p.Vc.sb_tile_off + (size_t)bh * tiles_cap : nullptr;
    const uint32_t main_off = (uint32_t)(col * mrb + grp * NB), aux_off = (uint32_t)(col * arb + grp * ABYTES);
    const uint32_t scale_off = (uint32_t)(4 * grp);
    const int k_count = FLAGS ? (int)min((int64_t)max(w_kcount, 0), p.Kc.sb_cap) : 0;
    const int v_count = FLAGS ? (int)min((int64_t)max(w_vcount, 0), p.Vc.sb_cap) : 0;
    const char *k_side = FLAGS ? (const char *)p.Kc.sideband + (size_t)bh * p.Kc.sb_cap * 8 : nullptr;
    const char *v_side = FLAGS ? (const char *)p.Vc.sideband + (size_t)bh * p.Vc.sb_cap * 8 : nullptr;
    const char *k_coord = FLAGS ? (const char *)p.Kc.sb_coord + (size_t)bh * p.Kc.sb_cap * 2 : nullptr;
    const char *v_coord = FLAGS ? (const char *)p.Vc.sb_coord + (size_t)bh * p.Vc.sb_cap * 2 : nullptr;
    const uint32_t v_cap1 = FLAGS ? (uint32_t)(p.Vc.sb_cap - 1) : 0u;
    const uint32_t k_cap2 = FLAGS ? (uint32_t)(p.Kc.sb_cap - 2) : 0u;        // sb_cap >= 2 is checked at launch

    auto load_super = [&](int t0, FastTile<NW, AB, FLAGS, NH> &s) {
        // in the order the half-steps consume them: K, then V, of tokens 0..31, then the same of tokens 32..63
#pragma unroll
        for (int hh = 0; hh < NH; hh++) {
            const int th = t0 + 32 * hh;
            const uint8_t *kb = k_rows + (size_t)th * mrb, *vb = v_rows + (size_t)th * mrb;
            HalfTile<NW, AB, FLAGS> &h = s.h[hh];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                load_bytes<NB>(kb + main_off + u * 16 * mrb, h.kw[u]);
                if (AB) h.kaux[u] = load_small<ABYTES>(ka_rows + (size_t)th * arb + aux_off + u * 16 * arb);
                h.ks[u] = *reinterpret_cast<const uint2 *>(ks_plane + th + scale_off + 16 * u);
            }
#pragma unroll
            for (int u = 0; u < 2; u++) {
                load_bytes<NB>(vb + main_off + u * 16 * mrb, h.vw[u]);
                if (AB) h.vaux[u] = load_small<ABYTES>(va_rows + (size_t)th * arb + aux_off + u * 16 * arb);
                h.vs[u] = *reinterpret_cast<const uint2 *>(vs_plane + th + scale_off + 16 * u);
            }
        }
    };

    // Tile offsets of one half-step, in two parts.  The loads (of wave-uniform addresses) are requested two half-steps
    // ahead; their clamping happens only when flags_ready has let them through at the end of a half-step: placed right
    // behind the loads it would wait for them with every later load in flight.
    // The offsets are read through the constant address space (nothing writes them while this kernel runs), which
    // makes them scalar loads: as vector loads of one address for all lanes, the six of a half-step took a memory
    // pipeline slot each and came back through v_readfirstlane (config 4: 10 % of the launch).
    typedef const int32_t __attribute__((address_space(4))) *const_i32_ptr;
    const const_i32_ptr k_toff_c = (const_i32_ptr)(uintptr_t)k_toff, v_toff_c = (const_i32_ptr)(uintptr_t)v_toff;
    auto load_flags = [&](int th, FlagTile &f) {
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const int tc = min((th >> 4) + i, tiles_cap1);
            f.koff[i] = k_toff_c[tc];
            f.voff[i] = v_toff_c[tc];
        }
    };
    auto flags_ready = [&](int th, FlagTile &f) {
#pragma unroll
        for (int i = 0; i < 3; i++) {
            asm volatile("" : "+s"(f.koff[i]), "+s"(f.voff[i]));        // this is where the scalar loads are waited for
        }
        // tiles not written yet hold INT32_MAX, and so does the slot after the last tile: the count bounds them
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const bool in = (th >> 4) + i <= tiles_cap1;
            f.koff[i] = min(in ? f.koff[i] : 0x7fffffff, k_count);
            f.voff[i] = min(in ? f.voff[i] : 0x7fffffff, v_count);
        }
        // a tile has at most 16 n entries: bounds the walk if the caller's offsets are inconsistent
#pragma unroll
        for (int i = 1; i < 3; i++) {
            f.koff[i] = min(f.koff[i], f.koff[i - 1] + 16 * n);
            f.voff[i] = min(f.voff[i], f.voff[i - 1] + 16 * n);
        }
    };

    // Every load of the loop is issued unconditionally (clamped addresses): a load inside a branch would make the
    // compiler's wait counts assume it was not issued, and the waits would then cover the next tile's prefetch.
    // K side.  The sideband entries of a half-step are a contiguous range known from three tile offsets, so no
    // flag is read: a batch of eight entries is the reduction dimension of one MFMA per tile,
    //   so[token][column] += sum over entries e of the batch, i < 4:  [token(e) == token] x_e[i] * Q[column][4 chunk(e) + i],
    // A = the lane's two entries where their token is the lane's row (else zero), B = the Q chunks they meet (LDS).
    // The lane's two entries are neighbours in the list: one 16-byte load of the chunks (8-byte aligned) and one 4-byte
    // load of the coordinates (2-byte aligned), at 32-bit byte offsets from wave-uniform bases (sb_cap < 2^28 is checked
    // at launch).  The pair is clamped to the last pair of the list's storage: an entry that is the very last slot of
    // a full list then arrives in the upper half.  (A wave-uniform branch to an unclamped variant measures slower.)
    // (The loaded words are kept as they come and put right by k_fix_x / k_fix_cc where they are used: touching them here would
    // make the request wait for its own data, and for every request before it.)
    auto k_load = [&](int bs, uint4v &x, uint32_t &cc) {
        const uint32_t ec = min((uint32_t)bs + 2u * (uint32_t)grp, k_cap2);
        x = *reinterpret_cast<const uint4v_a8 *>(k_side + ec * 8u);
        cc = *reinterpret_cast<const uint32_a2 *>(k_coord + ec * 2u);
    };
    auto k_fix_cc = [&](int bs, uint32_t cc) { return (uint32_t)bs + 2u * (uint32_t)grp > k_cap2 ? cc >> 16 : cc; };
    auto k_fix_x = [&](int bs, uint4v X, uint2 (&x)[2]) {
        const bool up = (uint32_t)bs + 2u * (uint32_t)grp > k_cap2;
        x[0] = uint2{up ? X[2] : X[0], up ? X[3] : X[1]};
        x[1] = uint2{X[2], X[3]};
    };
    auto k_issue = [&](const FlagTile &f, KPre<kKPre> &k) {
#pragma unroll
        for (int i = 0; i < 3; i++) k.off[i] = f.koff[i];
#pragma unroll
        for (int bq = 0; bq < kKPre; bq++) k_load(k.off[0] + 8 * bq, k.x[bq], k.cc[bq]);
    };
    constexpr int kVPre = CPL >= 8 ? 2 : 1;
    auto v_load = [&](int bs, uint2 &x, uint32_t &cc) {
        const uint32_t e = min((uint32_t)bs + (uint32_t)col, v_cap1);
        x = *reinterpret_cast<const uint2 *>(v_side + e * 8u);
        cc = *reinterpret_cast<const uint16_t *>(v_coord + e * 2u);
    };
    auto v_issue = [&](const FlagTile &f, VPre<kVPre> &v) {
#pragma unroll
        for (int i = 0; i < 3; i++) v.off[i] = f.voff[i];
#pragma unroll
        for (int bq = 0; bq < kVPre; bq++) v_load(v.off[0] + 16 * bq, v.x[bq], v.cc[bq]);
    };
    // sideband requests of one half-step
    auto issue_all = [&](const FlagTile &f, KPre<kKPre> &k, VPre<kVPre> &v) {
        k_issue(f, k);
        v_issue(f, v);
    };
    KPre<kKPre> kc = {};
    VPre<kVPre> vc = {};
    FastTile<NW, AB, FLAGS, NH> cur;
    FlagTile f0 = {}, f1 = {};
    uint2 q_raw[NCG][CPL];      // the query rows as stored
    {
        // unconditional (a wavefront without a range reads a valid tile it never uses): no branch, so the waits for the
        // table loads below count these loads as issued
        const int t_first = min(t_begin, (int)p.t_cap - 32);
        if (FLAGS) load_flags(t_first, f0);
        // Requests go out in the order their data is used, since they come back in that order and a wait for one is a
        // wait for all before it: tables (requested at the very start), query rows, first tile, its sideband entries.
        // All 16 lanes of a row load (columns past the end read column 0 again and are cleared below): unconditional,
        // so that the waits count them.
#pragma unroll
        for (int cgi = 0; cgi < NCG; cgi++) {
            const uint16_t *qp = (const uint16_t *)p.Q + b * p.qsb + hq[cgi] * p.qsh + (int64_t)tq[cgi] * p.qst + grp * CPL * 4;
#pragma unroll
            for (int j = 0; j < CPL; j++) q_raw[cgi][j] = *reinterpret_cast<const uint2 *>(qp + 4 * j);
        }
        load_super(t_first, cur);
#ifdef HQMQ_STAMPS
        ph_[2] = __builtin_amdgcn_s_memrealtime();      // first tile requested
#endif
        if constexpr (FLAGS) {
            // the first half-step's sideband entries are requested here, behind its tile: they travel while the tables
            // are filled (requested behind the barrier, they were the last thing the first half-step waited for)
            flags_ready(t_first, f0);
            issue_all(f0, kc, vc);          // unconditional (clamped addresses): a wavefront without a range reads entries it never uses
            load_flags(t_begin + TS < t_end ? t_begin + TS : t_first, f1);        // made ready behind the barrier
        }
    }
#ifdef HQMQ_STAMPS
    ph_[1] = __builtin_amdgcn_s_memrealtime();      // the first half-step's entries requested
#endif
    // Plain variants keep two half-steps in flight; the second is requested right behind the first (both queue
    // behind the table loads, which were requested at the very start).
    auto readable = [&](int t) { return min(t, (int)p.t_cap - 32); };
    FastTile<NW, AB, FLAGS, NH> tb;
    if constexpr (!FLAGS) load_super(readable(t_begin + TS < t_end ? t_begin + TS : t_begin), tb);
    half4 ident;                        // B operand of the transposing MFMA: the 16x16 identity
#pragma unroll
    for (int e = 0; e < 4; e++) ident[e] = (_Float16)((4 * grp + e) == col ? 1.f : 0.f);
    // bf16 caches: the verbatim sideband chunks (and the Q copy they meet) go into bf16 MFMAs as they are stored,
    // which saves their conversion to fp16 (6 VALU per chunk); the products are exact either way
    constexpr bool kBfEntries = FLAGS && DT == HQMQ_BF16;
    short4v ident_bf;
#pragma unroll
    for (int e = 0; e < 4; e++) ident_bf[e] = (short)((4 * grp + e) == col ? 0x3F80 : 0);

    {
        if constexpr (PS) {
            // tables multiplied out: codeword * rq for rq = 0..7 at (rq << 10 | idx) * 8 (K <= 1024: FU * NT pairs cover it)
#pragma unroll
            for (int u = 0; u < FU; u++) {
                const int k = threadIdx.x + u * NT;
                const uint4v hk = pair_to_half<DT>(tk[u]), hv = pair_to_half<DT>(tv[u]);
#pragma unroll
                for (int rq = 0; rq < 8; rq++) {
                    const half2v f = half2v{(_Float16)(float)rq, (_Float16)(float)rq};
                    auto mul = [&](uint32_t w) { return __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2v, w) * f); };
                    if (k < Kk2) reinterpret_cast<uint4v *>(ktab)[rq * 512 + k] = uint4v{mul(hk[0]), mul(hk[1]), mul(hk[2]), mul(hk[3])};
                    if (k < Kv2) reinterpret_cast<uint4v *>(vtab)[rq * 512 + k] = uint4v{mul(hv[0]), mul(hv[1]), mul(hv[2]), mul(hv[3])};
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < FU; u++) {
                const int k = threadIdx.x + u * NT;
                if (k < Kk2) store_pair<DT, F8>(ktab, k, tk[u]);
                if (k < Kv2) store_pair<DT, F8>(vtab, k, tv[u]);
            }
        }
    }
    if (FLAGS && threadIdx.x >= 64 && threadIdx.x < 100) {
        const uint32_t w = threadIdx.x - 64, row = w >> 2, d = w & 3;
        // the selector rows carry qmax instead of 1: the gathered probabilities come out scaled for the verbatim
        // chunks (whose 1 / qmax is applied with everything else in the epilogue) at no cost
        const uint32_t one = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)(float)p.qmax);
        reinterpret_cast<uint32_t *>(lds_tab)[SELOFF / 4 + w] = (row < 8 && (row >> 1) == d) ? one << (16 * (row & 1)) : 0u;
    }
    half8 qf[NCG][CPL / 2];
#pragma unroll
    for (int cgi = 0; cgi < NCG; cgi++) {
#pragma unroll
        for (int j = 0; j < CPL / 2; j++) {
            const half4 z = half4{0, 0, 0, 0};
            qf[cgi][j] = cat8(col_ok[cgi] ? chunk_to_half<DT>(q_raw[cgi][2 * j]) : z, col_ok[cgi] ? chunk_to_half<DT>(q_raw[cgi][2 * j + 1]) : z);
        }
    }
    if (FLAGS && wave == 0) {       // every wavefront of the block has the same 16 columns
#pragma unroll
        for (int jj = 0; jj < CPL / 2; jj++) {
            uint4v q8 = __builtin_bit_cast(uint4v, qf[0][jj]);
            if constexpr (kBfEntries) {         // the stored bf16 values
                const uint2 lo = col_ok[0] ? q_raw[0][2 * jj] : uint2{0, 0}, hi = col_ok[0] ? q_raw[0][2 * jj + 1] : uint2{0, 0};
                q8 = uint4v{lo.x, lo.y, hi.x, hi.y};
            }
            const int c0 = grp * CPL + 2 * jj;
            lds_tab[QOFF / 8 + c0 * 16 + col] = uint2{q8[0], q8[1]};
            lds_tab[QOFF / 8 + (c0 + 1) * 16 + col] = uint2{q8[2], q8[3]};
        }
    }
    // Progress slots of the wavefronts (see `publish` below), behind everything else the loop keeps in LDS
    const uint32_t prog_base = FLAGS ? (uint32_t)SELOFF + 192u : PS ? 2u * (uint32_t)kPsTabBytes : (uint32_t)kVTabOffset + (uint32_t)p.Vc.K * 8u;
    typedef int __attribute__((address_space(3))) *lds_i32_ptr;
    if (threadIdx.x < 16) *(lds_i32_ptr)(uintptr_t)(prog_base + 4u * threadIdx.x) = 0;
    if constexpr (MB == 16 && AB == 3 && IB == 13) {
        if (threadIdx.x < 64) {
            const uint32_t b6 = threadIdx.x;
            reinterpret_cast<uint32_t *>(lds_tab)[kAuxTabOffset / 4 + b6] = ((b6 & 7u) << 3) | ((b6 >> 3) << 19) | 0x64006400u;
        }
    }
#ifdef HQMQ_STAMPS
    const unsigned long long t_fill_ = __builtin_amdgcn_s_memrealtime();
#endif
    __syncthreads();
#ifdef HQMQ_STAMPS
    const unsigned long long t_bar_ = __builtin_amdgcn_s_memrealtime();
#endif

    // Scores are kept as v = S^T * rs (+ qmax * unscaled outlier part); the softmax argument is c_log2 * v.
    const float c = p.c_log2, qmaxf = (float)p.qmax;
    float m_run[NCG], l_run[NCG];
    float4v acc[NCG][CPL];
#pragma unroll
    for (int cgi = 0; cgi < NCG; cgi++) {
        m_run[cgi] = -INFINITY;
        l_run[cgi] = 0.f;
#pragma unroll
        for (int j = 0; j < CPL; j++) acc[cgi][j] = float4v{0.f, 0.f, 0.f, 0.f};
    }
    const float4v zero4 = float4v{0.f, 0.f, 0.f, 0.f};
    const half4 zero_h4 = half4{0, 0, 0, 0};
    // the Q chunks the lane's two entries meet (B operand rows), read from LDS well before the batch's MFMAs
    auto k_qrows = [&](uint32_t cc, uint2 (&q)[2]) {
        const uint32_t c0 = cc & (uint32_t)(n - 1), c1 = (cc >> 16) & (uint32_t)(n - 1);
        q[0] = __builtin_bit_cast(uint2, *(lds_u2_ptr)(uintptr_t)(QOFF + c0 * 128u + (uint32_t)col * 8u));
        q[1] = __builtin_bit_cast(uint2, *(lds_u2_ptr)(uintptr_t)(QOFF + c1 * 128u + (uint32_t)col * 8u));
    };
    auto k_batch = [&](const int (&off)[3], int bs, uint4v x_loaded, uint32_t cc_loaded, const uint2 (&q)[2], float4v (&so)[2]) {
        const int e0 = bs + 2 * grp;
        uint2 x[2];
        k_fix_x(bs, x_loaded, x);
        const uint32_t cc = k_fix_cc(bs, cc_loaded);
        // the row of the half-step (0..31) an entry belongs to; 64 for a slot behind the half-step's entries
        const uint32_t k0 = e0 < off[2] ? ((cc >> 8) & 15u) + (e0 >= off[1] ? 16u : 0u) : 64u;
        const uint32_t k1 = e0 + 1 < off[2] ? ((cc >> 24) & 15u) + (e0 + 1 >= off[1] ? 16u : 0u) : 64u;
        const uint2 zero_u2 = uint2{0u, 0u};
        half4 h0 = zero_h4, h1 = zero_h4;
        if constexpr (!kBfEntries) { h0 = chunk_to_half<DT>(x[0]); h1 = chunk_to_half<DT>(x[1]); }
        const half8 qq = cat8(__builtin_bit_cast(half4, q[0]), __builtin_bit_cast(half4, q[1]));
        // both tiles, no branch: the matrix unit is idle here and a skipped MFMA saves less than its test costs
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const bool v0 = k0 == (uint32_t)(col + 16 * u), v1 = k1 == (uint32_t)(col + 16 * u);
            if constexpr (kBfEntries) {
                const uint2 a0 = v0 ? x[0] : zero_u2, a1 = v1 ? x[1] : zero_u2;
                so[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, uint4v{a0.x, a0.y, a1.x, a1.y}),
                                                                __builtin_bit_cast(bf16x8, uint4v{q[0].x, q[0].y, q[1].x, q[1].y}),
                                                                so[u], 0, 0, 0);
            } else {
                so[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cat8(v0 ? h0 : zero_h4, v1 ? h1 : zero_h4), qq, so[u], 0, 0, 0);
            }
        }
    };
    struct KRows {
        uint2 q[kKPre][2];
    };
    auto k_prepare = [&](const KPre<kKPre> &k, KRows &r) {
#pragma unroll
        for (int bq = 0; bq < kKPre; bq++) k_qrows(k_fix_cc(k.off[0] + 8 * bq, k.cc[bq]), r.q[bq]);
    };
    auto k_apply = [&](const KPre<kKPre> &k, const KRows &r, float4v (&so)[2]) {
#pragma unroll
        for (int bq = 0; bq < kKPre; bq++)
            if (k.off[0] + 8 * bq < k.off[2]) k_batch(k.off, k.off[0] + 8 * bq, k.x[bq], k.cc[bq], r.q[bq], so);
        for (int bs = k.off[0] + 8 * kKPre; bs < k.off[2]; bs += 8) {      // more than the prefetched batches: rare
            uint4v x;
            uint2 q[2];
            uint32_t cc;
            k_load(bs, x, cc);
            k_qrows(k_fix_cc(bs, cc), q);
            k_batch(k.off, bs, x, cc, q, so);
        }
    };
    // V side, also from the entry list, sixteen entries of the half-step per batch (lane 16 * grp + col holds
    // entry `col`):
    //   Pg[e][column] = qmax P[token(e)][column] one 16x16x32 MFMA: A = qmax times the unit vector of the entry's token
    //                                            slot (LDS rows), B = the unscaled probabilities of the 32 tokens;
    //   for every chunk position j in use:       X_j^T by the transposing MFMA (A = the entry's chunk in the row
    //   acc[j] += X_j^T . Pg                     group that owns it, else zero), then one 16x16x16 MFMA over entries.
    // the selector row of the lane's entry (A operand of the MFMA that gathers the probabilities), read ahead of use
    auto v_sel = [&](const int (&off)[3], int bs, uint32_t cc) {
        const int e = bs + col;
        const uint32_t t = (cc >> 8) & 15u;
        const uint32_t slot = (e >= off[1] ? 4u : 0u) + (t & 3u);             // position among the row group's 8 tokens
        const bool mine = e < off[2] && (int)(t >> 2) == grp;
        return *(lds_u4_ptr)(uintptr_t)(SELOFF + (mine ? slot : 8u) * 16u);
    };
    auto v_batch = [&](const int (&off)[3], int bs, uint2 x, uint32_t cc, uint4v sel, half8 ppo) {
        const int e = bs + col;
        const uint32_t ch = cc & (uint32_t)(n - 1);
        const half4 pg = pack4(__builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, sel), ppo, zero4, 0, 0, 0));
        half4 h = zero_h4;
        if constexpr (!kBfEntries) h = chunk_to_half<DT>(x);
        const bool owner = e < off[2] && (int)(ch / CPL) == grp;
        const int jq = (int)(ch % CPL);
        // every chunk position, no test whether the batch meets it: straight-line code measures faster than skipping
        // the positions without an entry (the matrix unit is idle here, and a wave-uniform branch costs more than two MFMAs)
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            const bool mj = owner && jq == j;
            float4v tr;
            if constexpr (kBfEntries)
                tr = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4v, mj ? x : uint2{0u, 0u}), ident_bf, zero4, 0, 0, 0);
            else
                tr = __builtin_amdgcn_mfma_f32_16x16x16f16(mj ? h : zero_h4, ident, zero4, 0, 0, 0);
            acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x16f16(pack4(tr), pg, acc[0][j], 0, 0, 0);
        }
    };
    struct VSel {
        uint4v s[kVPre];
    };
    auto v_prepare = [&](const VPre<kVPre> &v, VSel &r) {
#pragma unroll
        for (int bq = 0; bq < kVPre; bq++) r.s[bq] = v_sel(v.off, v.off[0] + 16 * bq, v.cc[bq]);
    };
    auto v_apply = [&](const VPre<kVPre> &v, const VSel &r, half8 ppo) {
#pragma unroll
        for (int bq = 0; bq < kVPre; bq++)
            if (v.off[0] + 16 * bq < v.off[2]) v_batch(v.off, v.off[0] + 16 * bq, v.x[bq], v.cc[bq], r.s[bq], ppo);
        for (int bs = v.off[0] + 16 * kVPre; bs < v.off[2]; bs += 16) {     // more than the prefetched batches: rare
            uint2 x;
            uint32_t cc;
            v_load(bs, x, cc);
            v_batch(v.off, bs, x, cc, v_sel(v.off, bs, cc), ppo);
        }
    };

    // One half-step: 32 tokens (two tiles) through scores, online softmax and the V product.  A flagged chunk
    // carries radius code 0 in the main plane, so its decoded value is exactly zero and only the verbatim
    // value from the sideband contributes.
    auto half_step = [&](const HalfTile<NW, AB, FLAGS> &h, int th, const KPre<kKPre> &kc, const VPre<kVPre> &vc) {
        float4v sT[NCG][2], so[2] = {zero4, zero4};
        // the LDS operands of the outlier batches are requested first and used after the main products
        KRows kr;
        VSel vr;
        if constexpr (FLAGS) {
            k_prepare(kc, kr);
            v_prepare(vc, vr);
        }
        // every gather of the 32 K tokens is requested before the first one is used: the wavefront waits for LDS
        // once per half-step and tensor, not once per pair of chunks
        // (the variants that have no registers to spare keep the compiler's own interleaving of gathers and multiplies)
        half4 gk[2][CPL];
        half2v rk[2][CPL / 2];
        if constexpr (kBatchGathers) {
#pragma unroll
            for (int u = 0; u < 2; u++) gather_chunks<CPL, MB, AB, IB, NW, 0, F8>(h.kw[u], AB ? h.kaux[u] : 0u, idx_bits, gk[u], rk[u]);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            half4 a[CPL];
            if constexpr (!kBatchGathers) gather_chunks<CPL, MB, AB, IB, NW, 0, F8>(h.kw[u], AB ? h.kaux[u] : 0u, idx_bits, gk[u], rk[u]);
            scale_chunks<CPL, PS>(gk[u], rk[u], a);
#pragma unroll
            for (int cgi = 0; cgi < NCG; cgi++) {
                float4v s = zero4;
#pragma unroll
                for (int jj = 0; jj < CPL / 2; jj++)
                    s = __builtin_amdgcn_mfma_f32_16x16x32_f16(cat8(a[2 * jj], a[2 * jj + 1]), qf[cgi][jj], s, 0, 0, 0);
                if constexpr (!FLAGS) {
#pragma unroll
                    for (int e = 0; e < 4; e++) s[e] = scaled<DT>(s[e], e < 2 ? h.ks[u].x : h.ks[u].y, e & 1, 0.f);
                }
                sT[cgi][u] = s;
            }
        }
#ifdef HQMQ_STAMPS
        asm volatile("" ::"v"(sT[0][0]), "v"(sT[0][1]));
        PHASE(1);
#endif
        if constexpr (FLAGS) {
            k_apply(kc, kr, so);
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    sT[0][u][e] = scaled<DT>(sT[0][u][e], e < 2 ? h.ks[u].x : h.ks[u].y, e & 1, so[u][e] * qmaxf);
        }
#ifdef HQMQ_STAMPS
        asm volatile("" ::"v"(sT[0][0]), "v"(sT[0][1]));
        PHASE(2);
#endif
        // the V gathers fly while the softmax below keeps the vector unit busy
        half4 gv[2][CPL];
        half2v rv[2][CPL / 2];
        if constexpr (kBatchGathers) {
#pragma unroll
            for (int u = 0; u < 2; u++) gather_chunks<CPL, MB, AB, IB, NW, VTAB, F8>(h.vw[u], AB ? h.vaux[u] : 0u, idx_bits, gv[u], rv[u]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- mask (boundary half-steps only), online softmax, per column group ----
        const bool edge = !(th + 32 <= lim_min && th + 32 <= t_end && th >= col_start);
        half8 pp[NCG];
        half4 pTo[2];
#pragma unroll
        for (int cgi = 0; cgi < NCG; cgi++) {
            if (edge) {
#pragma unroll
                for (int u = 0; u < 2; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int t = th + 16 * u + 4 * grp + e;
                        if (!(t < col_lim[cgi] && t < t_end && t >= col_start)) sT[cgi][u][e] = -INFINITY;
                    }
            }
            float tmax = fmaxf(fmaxf(fmaxf(sT[cgi][0][0], sT[cgi][0][1]), fmaxf(sT[cgi][0][2], sT[cgi][0][3])),
                               fmaxf(fmaxf(sT[cgi][1][0], sT[cgi][1][1]), fmaxf(sT[cgi][1][2], sT[cgi][1][3])));
            tmax = row_max4(tmax);
            const float m_new = fmaxf(m_run[cgi], tmax);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            if (__builtin_amdgcn_ballot_w64(m_new != m_run[cgi]) != 0) {     // rescale only when some column's maximum moved
                const float alpha = __builtin_amdgcn_exp2f((m_run[cgi] - m_use) * c);
                l_run[cgi] *= alpha;
#pragma unroll
                for (int j = 0; j < CPL; j++) acc[cgi][j] = acc[cgi][j] * alpha;
                m_run[cgi] = m_new;
            }
            const float mc = -m_use * c;
            half4 pT[2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                float pe[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    pe[e] = __builtin_amdgcn_exp2f(fmaf(sT[cgi][u][e], c, mc));
                    l_run[cgi] += pe[e];
                }
                const half2v u01 = half2v{(_Float16)pe[0], (_Float16)pe[1]}, u23 = half2v{(_Float16)pe[2], (_Float16)pe[3]};
                const half2v p01 = u01 * scale_h2<DT>(h.vs[u].x);
                const half2v p23 = u23 * scale_h2<DT>(h.vs[u].y);
                pT[u] = half4{p01[0], p01[1], p23[0], p23[1]};
                if (FLAGS) pTo[u] = half4{u01[0], u01[1], u23[0], u23[1]};      // unscaled: the selector rows hold qmax
            }
            pp[cgi] = cat8(pT[0], pT[1]);
        }
#ifdef HQMQ_STAMPS
        asm volatile("" ::"v"(pp[0]));
        PHASE(3);
#endif
        // ---- O^T += V^T . P^T, both tiles in one MFMA (the 1/qmax of the radius is applied once, in the epilogue) ----
        if constexpr (kBatchGathers) __builtin_amdgcn_sched_barrier(0);
        half4 av[2][CPL];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            if constexpr (!kBatchGathers) gather_chunks<CPL, MB, AB, IB, NW, VTAB, F8>(h.vw[u], AB ? h.vaux[u] : 0u, idx_bits, gv[u], rv[u]);
            scale_chunks<CPL, PS>(gv[u], rv[u], av[u]);
        }
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            const float4v t0v = __builtin_amdgcn_mfma_f32_16x16x16f16(av[0][j], ident, zero4, 0, 0, 0);
            const float4v t1v = __builtin_amdgcn_mfma_f32_16x16x16f16(av[1][j], ident, zero4, 0, 0, 0);
            const half8 vt = cat8(pack4(t0v), pack4(t1v));
#pragma unroll
            for (int cgi = 0; cgi < NCG; cgi++) acc[cgi][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vt, pp[cgi], acc[cgi][j], 0, 0, 0);
        }
#ifdef HQMQ_STAMPS
        asm volatile("" ::"v"(acc[0][0]), "v"(acc[0][CPL - 1]));
        PHASE(4);
#endif
        if constexpr (FLAGS) v_apply(vc, vr, cat8(pTo[0], pTo[1]));
#ifdef HQMQ_STAMPS
        asm volatile("" ::"v"(acc[0][0]), "v"(acc[0][CPL - 1]));
        PHASE(5);
#endif
    };

    // The wavefronts that share a SIMD drift apart: the older one wins every tie for an issue slot, ends up several
    // half-steps ahead (config 4: 15 us at the end of a block) and leaves the younger to finish alone, with nothing
    // to overlap its waits.  Every wavefront publishes its position in LDS at the top of a half-step and reads its
    // SIMD neighbours' (wavefronts w, w + 4, w + 8 share a SIMD); at the end of the half-step it raises its priority
    // if one of them is ahead and drops it otherwise.
    int peer_pos = 0;
    auto publish = [&](int t0) {
        const int mine = t0 - 32 * wave;        // the same for all wavefronts at the same distance from the block's start
        *(lds_i32_ptr)(uintptr_t)(prog_base + 4u * (uint32_t)wave) = mine;
        peer_pos = *(lds_i32_ptr)(uintptr_t)(prog_base + 4u * (uint32_t)((wave + 4) % WV));
        if constexpr (WV > 8) peer_pos = max(peer_pos, *(lds_i32_ptr)(uintptr_t)(prog_base + 4u * (uint32_t)((wave + 8) % WV)));
    };
    // (A tie goes to the younger wavefront, w >= 4: at equal priority the hardware would give it to the older one.)
    auto rebalance = [&](int t0) {
        if (__builtin_amdgcn_readfirstlane(peer_pos) + (wave >= 4 ? 1 : 0) > t0 - 32 * wave) __builtin_amdgcn_s_setprio(3);
        else __builtin_amdgcn_s_setprio(0);
    };
    if constexpr (FLAGS) flags_ready(t_begin + TS < t_end ? t_begin + TS : min(t_begin, (int)p.t_cap - 32), f1);

    if constexpr (!FLAGS) {
        // ring of three tile buffers, every load unconditional (past the end the current tile is requested again)
        FastTile<NW, AB, FLAGS, NH> tc;
        int t0 = t_begin;
        if (t0 < t_end) {
            while (true) {
                load_super(readable(t0 + 2 * TS < t_end ? t0 + 2 * TS : t0), tc);
                publish(t0);
                half_step(cur.h[0], t0, kc, vc);
                rebalance(t0);
                t0 += TS;
                if (t0 >= t_end) break;
                load_super(readable(t0 + 2 * TS < t_end ? t0 + 2 * TS : t0), cur);
                publish(t0);
                half_step(tb.h[0], t0, kc, vc);
                rebalance(t0);
                t0 += TS;
                if (t0 >= t_end) break;
                load_super(readable(t0 + 2 * TS < t_end ? t0 + 2 * TS : t0), tb);
                publish(t0);
                half_step(tc.h[0], t0, kc, vc);
                rebalance(t0);
                t0 += TS;
                if (t0 >= t_end) break;
            }
        }
    }
    if constexpr (FLAGS) {
        // Outlier variants: one half-step in flight.  Two sets of buffers (tile, sideband entries, tile offsets) take
        // turns, written out as two half-steps per round of the loop: with one set handed on at the end of every
        // half-step (cur = nxt) the compiler copied some fifty registers per half-step.
        // Tile offsets travel two half-steps ahead, sideband entries one (their offsets were requested a step ago); past
        // the end the current tile is requested again.
        FastTile<NW, AB, FLAGS, NH> tile_b;
        KPre<kKPre> k_b = {};
        VPre<kVPre> v_b = {};
        FlagTile f2 = {};
        auto one = [&](int t0, const FastTile<NW, AB, FLAGS, NH> &tile_use, const KPre<kKPre> &k_use, const VPre<kVPre> &v_use,
                       FastTile<NW, AB, FLAGS, NH> &tile_load, KPre<kKPre> &k_load_to, VPre<kVPre> &v_load_to, const FlagTile &f_use,
                       FlagTile &f_load) {
            const bool more = t0 + TS < t_end, more2 = t0 + 2 * TS < t_end;
#ifdef HQMQ_STAMPS
            if (tl_ == 0) tl_ = t_loop_ = __builtin_amdgcn_s_memrealtime();
            n_steps_++;
#endif
            load_super(more ? t0 + TS : t0, tile_load);
            load_flags(more2 ? t0 + 2 * TS : t0, f_load);           // made ready at the end of this half-step
            issue_all(f_use, k_load_to, v_load_to);
            publish(t0);
            PHASE(0);
            half_step(tile_use.h[0], t0, k_use, v_use);
            rebalance(t0);
            if (more) flags_ready(more2 ? t0 + 2 * TS : t0, f_load);
            PHASE(6);
            return more;
        };
        if (t_begin < t_end) {
            int t0 = t_begin;
            while (true) {
                if (!one(t0, cur, kc, vc, tile_b, k_b, v_b, f1, f2)) break;
                t0 += TS;
                if (!one(t0, tile_b, k_b, v_b, cur, kc, vc, f2, f1)) break;
                t0 += TS;
            }
        }
    }
#ifdef HQMQ_STAMPS
    if constexpr (FLAGS) {
        if (lane == 0 && g_stamps) {
            unsigned long long *o = g_stamps + ((size_t)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * WV + wave) * 16;
#pragma unroll
            for (int i = 0; i < 7; i++) o[i] = ph_[i];
            o[7] = (unsigned long long)n_steps_;
            o[8] = t_in_;                   // entry, first half-step, last half-step done (the block's merge follows)
            o[9] = t_loop_;
            o[10] = __builtin_amdgcn_s_memrealtime();
            // where the block ran: HW_ID (bits 8-11 CU, 12 SH, 13-15 SE) and XCC_ID (bits 0-3)
            o[11] = (unsigned long long)__builtin_amdgcn_s_getreg(((32 - 1) << 11) | 4) |
                    ((unsigned long long)__builtin_amdgcn_s_getreg(((4 - 1) << 11) | 20) << 32);
            o[12] = (unsigned long long)b;
            o[14] = t_fill_;                // own share of the tables stored, barrier passed
            o[15] = t_bar_;
        }
    }
#endif

    // ---- merge the block's waves through LDS: rows of [d_h accumulators, m, l, pad], one column group at a time ----
    constexpr int RS = d_h + 4;
    float *red = reinterpret_cast<float *>(lds_tab);            // [wave][16 cols][RS]
    const float inv_qmax = p.inv_qmax;
#pragma unroll
    for (int cgi = 0; cgi < NCG; cgi++) {
        const int cg = cg0 + cgi;
        const float l_tot = row_sum4(l_run[cgi]);
        __syncthreads();
        const int ncols = min(16, p.Tq * G - cg * 16);          // <= 0 for a column group past the end
        if (col < ncols) {                                      // padding columns are never read back
            float *wp = red + ((size_t)wave * 16 + col) * RS;
            if (grp == 0) { wp[d_h] = m_run[cgi]; wp[d_h + 1] = l_tot; }
#pragma unroll
            for (int j = 0; j < CPL; j++) *reinterpret_cast<float4v *>(wp + grp * CPL * 4 + 4 * j) = acc[cgi][j];
        }
        __syncthreads();
        for (int o = threadIdx.x; o < ncols * d_h; o += NT) {
            const int cc = o / d_h, e = o - cc * d_h;
            const int ci = cg * 16 + cc;
            float m = -INFINITY;
#pragma unroll
            for (int w = 0; w < WV; w++) m = fmaxf(m, red[((size_t)w * 16 + cc) * RS + d_h]);
            float l = 0.f, a = 0.f;
            if (m > -INFINITY) {
#pragma unroll
                for (int w = 0; w < WV; w++) {
                    const float *q = red + ((size_t)w * 16 + cc) * RS;
                    const float f = __builtin_amdgcn_exp2f((q[d_h] - m) * c);
                    l = fmaf(q[d_h + 1], f, l);
                    a = fmaf(q[e], f, a);
                }
            }
            const int tq2 = (int)fast_div((unsigned)ci, (unsigned)G, p.m_G), hq2 = hkv * G + (ci - tq2 * G);
            if (p.n_splits == 1) {
                store_any(p.O, DT, b * p.osb + hq2 * p.osh + (int64_t)tq2 * p.ost + e, l > 0.f ? a * inv_qmax / l : 0.f);
            } else {
                // partials carry the maximum in softmax units (base-2 exponent) and acc already divided by qmax
                float *wp = p.ws + ((((size_t)b * p.Hq + hq2) * p.Tq + tq2) * p.n_splits + sp) * (size_t)(d_h + kPartialHead);
                if (e == 0) { wp[0] = m * c; wp[1] = l; }
                wp[kPartialHead + e] = a * inv_qmax;
            }
        }
    }
#ifdef HQMQ_STAMPS
    if constexpr (FLAGS) {
        if (lane == 0 && g_stamps)
            g_stamps[((size_t)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * WV + wave) * 16 + 13] = __builtin_amdgcn_s_memrealtime();
    }
#endif
}

// ---------------------------------------------------------------------------------------------------------------
// Plain 16+0 caches at d_h 128 with tables of at most 2304 codewords (s96_r4 and smaller): the variant whose loads
// all land in LDS (global_load_lds: the data goes from memory to LDS without passing through registers).  Tables,
// the query rows and the first half-step of every wavefront are requested in the prologue; from then on a wavefront
// asks for its next half-step when the current one has arrived and its words have been read out of the slot, so one
// half-step per wavefront is in flight while one is being worked on.  Measured on config 2 at 32k, planes read cold
// from HBM: asking for more ahead (two or three half-steps, before or behind the barrier) floods the memory system,
// and the half-steps that are needed first then arrive behind later ones (first half-step in at 4.4 us median and
// 8.2 us at worst with three ahead, 3.2 / 4.4 us with one); kernel 15.0 - 15.9 us with two or three ahead, 13.2 us
// with one (the register-tile kernel, which keeps two ahead in 40 registers: 15.0 us).
// No tile lives in registers while in flight (111 registers against 145 - 256).  The compiler neither sees these
// loads nor counts them: every wait is written by hand (s_waitcnt vmcnt(n) lets the n youngest requests stay
// outstanding; requests complete in order), and the kernel has no other vector loads before its epilogue.
// LDS: K table at 0, V table at 18432, 4 KB of query rows, then per wavefront two slots of
// [256 B scales: K tokens 0..31, V tokens 0..31, the same again][K rows of 32 tokens, 2 KB][V rows, 2 KB].
constexpr int kLdVTab = 2304 * 8;
constexpr int kLdQ = 2 * kLdVTab;
constexpr int kLdSlot0 = kLdQ + 4096;
constexpr int kLdSlotBytes = 256 + 4096;

template <int N>
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// wait until at most `groups` (0..3) groups of five requests are outstanding
__device__ __forceinline__ void wait_groups(int groups) {
    if (groups >= 3) wait_vm<15>();
    else if (groups == 2) wait_vm<10>();
    else if (groups == 1) wait_vm<5>();
    else wait_vm<0>();
}
__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t *)(((uint64_t)hi << 32) | lo);
}
// 64 lanes x 16 bytes from base + voff (+ the instruction's offset, which counts for both sides) to LDS at m0 + 16 * lane
__device__ __forceinline__ void lds_load16(uint32_t lds_base, const uint8_t *base, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(base) : "memory");
}
__device__ __forceinline__ void lds_load16_addr(uint32_t lds_base, const uint8_t *addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(addr) : "memory");
}
__device__ __forceinline__ uint4v lds_read16(uint32_t a) { return *(lds_u4_ptr)(uintptr_t)a; }
__device__ __forceinline__ uint2 lds_read8(uint32_t a) { return __builtin_bit_cast(uint2, *(lds_u2_ptr)(uintptr_t)a); }


constexpr int kLdDepth = 2;

template <int DT, int IB, int WV>
__global__ __launch_bounds__(WV * 64) void attn_lds_kernel(AttnParams p) {
    constexpr int CPL = 8, NW = 4, d_h = 128, mrb = 64;
    extern __shared__ uint2 lds_tab[];
#ifdef HQMQ_STAMPS
    unsigned long long st_[16] = {};
#endif
    STAMP(0);
    // Everything the first requests need is read from the argument block in one go (the empty asm below is where
    // all of it has to be there): read where it is used, every group of arguments costs its own round trip.
    // The grid is (n_splits, column groups, B * Hkv): taken from the arguments, which spares the dispatch packet.
    const unsigned gx = (unsigned)p.n_splits, gy = (unsigned)p.n_cg, gz = (unsigned)(p.B * p.Hkv);
    const int Hkv = p.Hkv, remap = p.xcd_remap;
    const unsigned m_gz = p.m_gz, m_gx = p.m_gx, m_hkv = p.m_hkv;
    const int32_t *order_p = p.batch_order, *len_p = p.kv_len, *start_p = p.kv_start;
    const uint8_t *kj = (const uint8_t *)p.Kc.joint, *vj = (const uint8_t *)p.Vc.joint;
    const int64_t kjsh = p.Kc.jsh, vjsh = p.Vc.jsh;
    const int KK = p.Kc.K, KV = p.Vc.K, Tkv = p.Tkv, Bn = p.B;
    asm volatile("" ::"s"(gx), "s"(gy), "s"(gz), "s"(Hkv), "s"(remap), "s"(m_gz), "s"(m_gx), "s"(m_hkv), "s"(order_p), "s"(len_p), "s"(start_p),
                 "s"(kj), "s"(vj), "s"(kjsh), "s"(vjsh), "s"(KK), "s"(KV), "s"(Tkv), "s"(Bn));
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    if (remap) {
        const unsigned lin = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
        const unsigned r = fast_div(lin, gz, m_gz);
        bz = (int)(lin - r * gz);
        by = (int)fast_div(r, gx, m_gx);
        bx = (int)(r - (unsigned)by * gx);
    }
    const int slot = (int)fast_div((unsigned)bz, (unsigned)Hkv, m_hkv), hkv = bz - slot * Hkv;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#ifdef HQMQ_STAMPS
    asm volatile("" ::"s"(hkv));
    STAMP(15);
#endif
    // the per-sequence words of ragged batches are read before the first request goes out: behind one, the wait for
    // such a word would also wait for every request in flight
    const int b = order_p ? min(max(uniform_word(order_p, slot), 0), Bn - 1) : slot;
    int kv_end = len_p ? uniform_word(len_p, b) : Tkv;
    kv_end = min(max(kv_end, 0), Tkv);
    const int kv_first = start_p ? max(uniform_word(start_p, b), 0) : 0;
    // ---- tables: 1 KB units dealt to the wavefronts round-robin, straight to their place in LDS ----
    {
        const uint32_t kbytes = (uint32_t)KK * 8u, vbytes = (uint32_t)KV * 8u;
        const uint8_t *ksrc = uniform_ptr(kj + (size_t)hkv * kjsh * 2);
        const uint8_t *vsrc = uniform_ptr(vj + (size_t)hkv * vjsh * 2);
        const int ku = (int)((kbytes + 1023u) >> 10), nu = ku + (int)((vbytes + 1023u) >> 10);
        for (int u = wave; u < nu; u += WV) {
            const bool isv = u >= ku;
            const uint32_t uu = (uint32_t)(isv ? u - ku : u);
            const uint32_t off = min(uu * 1024u + (uint32_t)lane * 16u, (isv ? vbytes : kbytes) - 16u);      // past the end: the last pair again
            lds_load16((isv ? (uint32_t)kLdVTab : 0u) + uu * 1024u, isv ? vsrc : ksrc, off);
        }
    }
    STAMP(1);
    const int bh = b * p.Hkv + hkv;
    const int cg = by, sp = bx;
    const int G = p.G;
    const int col = lane & 15, grp = lane >> 4;
    const int ncols = min(16, p.Tq * G - cg * 16);
    const int cidx = cg * 16 + col;
    const bool col_ok = col < ncols;
    const int tq = col_ok ? (int)fast_div((unsigned)cidx, (unsigned)G, p.m_G) : 0;
    int col_lim, blk_lim, lim_min;
    {
        int64_t lim64 = kv_end;
        if (p.causal) lim64 = min(lim64, (int64_t)tq + p.causal_offset + 1);
        if (!col_ok || lim64 < 0) lim64 = 0;
        col_lim = (int)lim64;
        blk_lim = col_lim;
        lim_min = col_ok ? col_lim : 0x7fffffff;
    }
    if (p.causal) {
        for (int o = 1; o < 16; o <<= 1) {
            blk_lim = max(blk_lim, __shfl_xor(blk_lim, o));
            lim_min = min(lim_min, __shfl_xor(lim_min, o));
        }
        blk_lim = __builtin_amdgcn_readfirstlane(blk_lim);
        lim_min = __builtin_amdgcn_readfirstlane(lim_min);
    } else {
        blk_lim = lim_min = kv_end;
    }
    const int col_start = min(kv_first, blk_lim);
    const int blk_lo = col_start / kSuper * kSuper;
    int per_split = (int)fast_div((unsigned)(blk_lim - blk_lo + p.n_splits - 1), (unsigned)p.n_splits, p.m_splits);
    per_split = (per_split + kSuper - 1) / kSuper * kSuper;
    const int b_begin = min(blk_lo + sp * per_split, blk_lim), b_end = min(blk_lim, b_begin + per_split);
    constexpr int TS = 32 * WV;
    const int t_begin = min(b_begin + wave * 32, b_end), t_end = b_end;
    const int n_hs = __builtin_amdgcn_readfirstlane(t_begin < t_end ? (t_end - t_begin + TS - 1) / TS : 0);
    const size_t plane_row0 = (size_t)bh * p.t_cap;
    const int idx_bits = p.idx_bits;
    // instruction offsets count for the memory and the LDS side alike: the bases are moved back by the slot offsets
    const uint8_t *k_rows = p.Kc.main_plane + plane_row0 * mrb - 256;
    const uint8_t *v_rows = p.Vc.main_plane + plane_row0 * mrb - 2304;
    const uint32_t main_off = (uint32_t)(col * mrb + grp * 16);
    // scales: lanes 0..15 fetch the K scales of tokens 2 lane, 2 lane + 1, lanes 16..31 the V scales; the upper half repeats
    const uint8_t *sc_lane = (lane & 16) ? (const uint8_t *)((const uint16_t *)p.Vc.scale_plane + b * p.Vc.ssb + hkv * p.Vc.ssh)
                                         : (const uint8_t *)((const uint16_t *)p.Kc.scale_plane + b * p.Kc.ssb + hkv * p.Kc.ssh);
    sc_lane += 4 * (lane & 15);
    const uint32_t slot_base = (uint32_t)(kLdSlot0 + wave * kLdDepth * kLdSlotBytes);
    auto request = [&](int th, uint32_t slot_lds) {
        const uint8_t *kb = uniform_ptr(k_rows + (size_t)th * mrb), *vb = uniform_ptr(v_rows + (size_t)th * mrb);
        const uint8_t *sa = sc_lane + 2 * (size_t)th;
        asm volatile("s_mov_b32 m0, %0\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:256\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:1280\n\t"
                     "global_load_lds_dword %1, off\n\t"
                     "global_load_lds_dwordx4 %2, %4 offset:2304\n\t"
                     "global_load_lds_dwordx4 %2, %4 offset:3328"
                     ::"s"(slot_lds), "v"(sa), "v"(main_off), "s"(kb), "s"(vb) : "memory");
    };
    // ---- query rows (first wavefront): column c of the block at kLdQ + 256 c, raw 16-bit values ----
    if (wave == 0) {
        for (int i = 0; 4 * i < ncols; i++) {       // four columns per request; a decode step of G <= 4 heads takes one
            const int c = min(4 * i + (lane >> 4), ncols - 1);              // lanes past the last real column repeat it (never read)
            const int ci = cg * 16 + c;
            const int tqc = (int)fast_div((unsigned)ci, (unsigned)G, p.m_G), hqc = hkv * G + (ci - tqc * G);
            const uint8_t *qa = (const uint8_t *)((const uint16_t *)p.Q + b * p.qsb + hqc * p.qsh + (int64_t)tqc * p.qst) + 16 * (lane & 15);
            lds_load16_addr((uint32_t)(kLdQ + 1024 * i), qa);
        }
    }
    // the first half-step; the later ones are requested from inside the loop, one ahead
    if (n_hs > 0) request(t_begin, slot_base);
    STAMP(2);
    half4 ident;
#pragma unroll
    for (int e = 0; e < 4; e++) ident[e] = (_Float16)((4 * grp + e) == col ? 1.f : 0.f);
    wait_groups(n_hs > 0 ? 1 : 0);            // tables (and query rows) in: only the tile request may still be outstanding
    STAMP(3);
    asm volatile("s_barrier" ::: "memory");
    if constexpr (DT != HQMQ_F16) {
        // the tables landed in the cache dtype: converted to fp16 in place, two codewords per thread and round
        for (int k = threadIdx.x; k < (2 * kLdVTab) / 16; k += WV * 64) {
            const uint4v w = pair_to_half<DT>(lds_read16((uint32_t)k * 16u));
            *(uint4v __attribute__((address_space(3))) *)(uintptr_t)((uint32_t)k * 16u) = w;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);         // lgkmcnt(0): the stores are in LDS
        asm volatile("s_barrier" ::: "memory");
    }
    STAMP(4);
    half8 qf[CPL / 2];
#pragma unroll
    for (int j = 0; j < CPL / 2; j++) {
        const uint4v w = lds_read16((uint32_t)(kLdQ + col * 256 + grp * 64 + 16 * j));
        const half4 lo = chunk_to_half<DT>(uint2{w[0], w[1]}), hi = chunk_to_half<DT>(uint2{w[2], w[3]});
        const half4 z = half4{0, 0, 0, 0};
        qf[j] = cat8(col_ok ? lo : z, col_ok ? hi : z);
    }

    const float c = p.c_log2;
    float m_run = -INFINITY, l_run = 0.f;
    float4v acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};
    const float4v zero4 = float4v{0.f, 0.f, 0.f, 0.f};
    int ring = 0;
    for (int i = 0, th = t_begin; i < n_hs; i++, th += TS) {
        const uint32_t sl = slot_base + (uint32_t)ring * kLdSlotBytes, sl_next = slot_base + (uint32_t)(ring ^ 1) * kLdSlotBytes;
        ring ^= 1;
        // The hardware prefers the older of the two wavefronts of a SIMD, which then ends 1.7 us before the younger and
        // leaves it to finish alone.  Priority by work left (finer towards the end) lets the one that is behind go first,
        // so that the two finish together (kernel -0.3 us).
        const int left = n_hs - i;
        if (left >= 3) __builtin_amdgcn_s_setprio(3);
        else if (left == 2) __builtin_amdgcn_s_setprio(3);
        else __builtin_amdgcn_s_setprio(1);
        wait_groups(0);
#ifdef HQMQ_STAMPS
        { const unsigned long long t_ = __builtin_amdgcn_s_memrealtime();
          if (i == 0) st_[5] = t_; else if (i == 1) st_[7] = t_; else if (i == 2) st_[9] = t_; else if (i == 3) st_[11] = t_; }
#endif
        uint4v kw[2], vw[2];
        uint2 ks[2], vs[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            kw[u] = lds_read16(sl + 256u + 1024u * u + 16u * (uint32_t)lane);
            ks[u] = lds_read8(sl + 32u * u + 8u * (uint32_t)grp);
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            vw[u] = lds_read16(sl + 2304u + 1024u * u + 16u * (uint32_t)lane);
            vs[u] = lds_read8(sl + 64u + 32u * u + 8u * (uint32_t)grp);
        }
        // the words of this half-step are in registers: ask for the next one (into the other slot)
        asm volatile("" : "+v"(kw[0]), "+v"(kw[1]), "+v"(vw[0]), "+v"(vw[1]), "+v"(ks[0]), "+v"(ks[1]), "+v"(vs[0]), "+v"(vs[1]));
        if (i + 1 < n_hs) request(th + TS, sl_next);

        float4v sT[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            half4 g[CPL], a[CPL];
            half2v r[CPL / 2];
            const uint32_t w[NW] = {kw[u][0], kw[u][1], kw[u][2], kw[u][3]};
            gather_chunks<CPL, 16, 0, IB, NW, 0, false>(w, 0u, idx_bits, g, r);
            scale_chunks<CPL, false>(g, r, a);
            float4v s = zero4;
#pragma unroll
            for (int jj = 0; jj < CPL / 2; jj++) s = __builtin_amdgcn_mfma_f32_16x16x32_f16(cat8(a[2 * jj], a[2 * jj + 1]), qf[jj], s, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; e++) s[e] = scaled<DT>(s[e], e < 2 ? ks[u].x : ks[u].y, e & 1, 0.f);
            sT[u] = s;
        }
        const bool edge = !(th + 32 <= lim_min && th + 32 <= t_end && th >= col_start);
        if (edge) {
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int t = th + 16 * u + 4 * grp + e;
                    if (!(t < col_lim && t < t_end && t >= col_start)) sT[u][e] = -INFINITY;
                }
        }
        float tmax = fmaxf(fmaxf(fmaxf(sT[0][0], sT[0][1]), fmaxf(sT[0][2], sT[0][3])), fmaxf(fmaxf(sT[1][0], sT[1][1]), fmaxf(sT[1][2], sT[1][3])));
        tmax = row_max4(tmax);
        const float m_new = fmaxf(m_run, tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
            l_run *= alpha;
#pragma unroll
            for (int j = 0; j < CPL; j++) acc[j] = acc[j] * alpha;
            m_run = m_new;
        }
        const float mc = -m_use * c;
        half4 pT[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            float pe[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                pe[e] = __builtin_amdgcn_exp2f(fmaf(sT[u][e], c, mc));
                l_run += pe[e];
            }
            const half2v p01 = half2v{(_Float16)pe[0], (_Float16)pe[1]} * scale_h2<DT>(vs[u].x);
            const half2v p23 = half2v{(_Float16)pe[2], (_Float16)pe[3]} * scale_h2<DT>(vs[u].y);
            pT[u] = half4{p01[0], p01[1], p23[0], p23[1]};
        }
        const half8 pp = cat8(pT[0], pT[1]);
        if (left == 2) __builtin_amdgcn_s_setprio(2);
        else if (left == 1) __builtin_amdgcn_s_setprio(0);
        half4 av[2][CPL];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            half4 g[CPL];
            half2v r[CPL / 2];
            const uint32_t w[NW] = {vw[u][0], vw[u][1], vw[u][2], vw[u][3]};
            gather_chunks<CPL, 16, 0, IB, NW, kLdVTab, false>(w, 0u, idx_bits, g, r);
            scale_chunks<CPL, false>(g, r, av[u]);
        }
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            const float4v t0v = __builtin_amdgcn_mfma_f32_16x16x16f16(av[0][j], ident, zero4, 0, 0, 0);
            const float4v t1v = __builtin_amdgcn_mfma_f32_16x16x16f16(av[1][j], ident, zero4, 0, 0, 0);
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cat8(pack4(t0v), pack4(t1v)), pp, acc[j], 0, 0, 0);
        }
#ifdef HQMQ_STAMPS
        asm volatile("" ::"v"(acc[0]), "v"(acc[7]));
        { const unsigned long long t_ = __builtin_amdgcn_s_memrealtime();
          if (i == 0) st_[6] = t_; else if (i == 1) st_[8] = t_; else if (i == 2) st_[10] = t_; else if (i == 3) st_[12] = t_; }
#endif
    }

    // ---- merge the block's wavefronts through LDS: rows of [d_h accumulators, m, l, pad] ----
    constexpr int RS = d_h + 4, NT = WV * 64;
    float *red = reinterpret_cast<float *>(lds_tab);
    const float inv_qmax = p.inv_qmax;
    const float l_tot = row_sum4(l_run);
    __syncthreads();
    if (col < ncols) {
        float *wp = red + ((size_t)wave * 16 + col) * RS;
        if (grp == 0) { wp[d_h] = m_run; wp[d_h + 1] = l_tot; }
#pragma unroll
        for (int j = 0; j < CPL; j++) *reinterpret_cast<float4v *>(wp + grp * CPL * 4 + 4 * j) = acc[j];
    }
    __syncthreads();
    STAMP(13);
    for (int o = threadIdx.x; o < ncols * d_h; o += NT) {
        const int cc = o / d_h, e = o - cc * d_h;
        const int ci = cg * 16 + cc;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WV; w++) m = fmaxf(m, red[((size_t)w * 16 + cc) * RS + d_h]);
        float l = 0.f, a = 0.f;
        if (m > -INFINITY) {
#pragma unroll
            for (int w = 0; w < WV; w++) {
                const float *q = red + ((size_t)w * 16 + cc) * RS;
                const float f = __builtin_amdgcn_exp2f((q[d_h] - m) * c);
                l = fmaf(q[d_h + 1], f, l);
                a = fmaf(q[e], f, a);
            }
        }
        const int tq2 = (int)fast_div((unsigned)ci, (unsigned)G, p.m_G), hq2 = hkv * G + (ci - tq2 * G);
        if (p.n_splits == 1) {
            store_any(p.O, DT, b * p.osb + hq2 * p.osh + (int64_t)tq2 * p.ost + e, l > 0.f ? a * inv_qmax / l : 0.f);
        } else {
            float *wp = p.ws + ((((size_t)b * p.Hq + hq2) * p.Tq + tq2) * p.n_splits + sp) * (size_t)(d_h + kPartialHead);
            if (e == 0) { wp[0] = m * c; wp[1] = l; }
            wp[kPartialHead + e] = a * inv_qmax;
        }
    }
#ifdef HQMQ_STAMPS
    STAMP(14);
    if (lane == 0 && g_stamps) {
        unsigned long long *o = g_stamps + ((size_t)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * WV + wave) * 16;
#pragma unroll
        for (int i = 0; i < 16; i++) o[i] = st_[i];
    }
#endif
}

template <int DT, int IB, int WV>
static int launch_lds_waves(const AttnParams &p, dim3 grid, hipStream_t st, const LaunchTiming &tm) {
    constexpr size_t kTiles = (size_t)kLdSlot0 + (size_t)WV * kLdDepth * kLdSlotBytes;
    constexpr size_t kMerge = (size_t)WV * 16 * (128 + 4) * sizeof(float);
    constexpr size_t shmem = kTiles > kMerge ? kTiles : kMerge;
    static_assert(shmem <= 160 * 1024, "LDS of one CU");
    auto kern = attn_lds_kernel<DT, IB, WV>;
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
    launch_timed(kern, grid, dim3(WV * 64), shmem, st, tm, p);
    return hip_status(hipGetLastError());
}
template <int DT, int IB>
static int launch_lds(const AttnParams &p, dim3 grid, hipStream_t st, const LaunchTiming &tm) {
    // (four-wavefront blocks for short ranges measured no faster: 8.9 against 8.7 us per step at 4k tokens)
    return launch_lds_waves<DT, IB, kFastWaves>(p, grid, st, tm);
}

template <int CPL, int MB, int AB, int IB, int DT, int WV = kFastWaves, int NCG = 1, bool F8 = false>
static int launch_one(const AttnParams &p, bool flags, dim3 grid, hipStream_t st, const LaunchTiming &tm) {
    if (NCG > 1) grid.y = (grid.y + NCG - 1) / NCG;
    // LDS: K table at 0, V table at kVTabOffset; reused afterwards for the cross-wave merge [wave][16][d_h + 4] floats
    constexpr bool PS = is_prescaled(CPL, MB, AB, IB);
    size_t shmem = flags ? (size_t)sel_offset(PS) + 192 : PS ? (size_t)2 * kPsTabBytes : (size_t)kVTabOffset + (size_t)p.Vc.K * 8;
    shmem += 64;        // the wavefronts' progress slots
    const size_t merge = (size_t)WV * 16 * (16 * CPL + 4) * sizeof(float);     // WV >= the wavefronts actually launched
    if (shmem < merge) shmem = merge;
    constexpr int WF = CPL == 4 ? WV : kFastWaves;      // outlier variants fit three wavefronts per SIMD only at d_h 64
    auto kern = flags ? attn_fast_kernel<CPL, MB, AB, IB, DT, true, WF, 1, F8> : attn_fast_kernel<CPL, MB, AB, IB, DT, false, WV, NCG, F8>;
    if (shmem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    launch_timed(kern, grid, dim3((flags ? WF : WV) * 64), shmem, st, tm, p);
    return hip_status(hipGetLastError());
}

template <int CPL, int DT>
static int launch_layout(const AttnParams &p, int mb, bool flags, dim3 grid, hipStream_t st, const LaunchTiming &tm, bool *handled) {
    if (p.Kc.K > kVTabOffset / 8 || p.Vc.K > kVTabOffset / 8) return HQMQ_OK;     // tables beyond the fixed LDS slots
    // the kernels divide by multiplication only (fast_div): sizes for which a multiplier cannot be promised (index times
    // divisor beyond 2^32: millions of tokens times thousands of splits) stay with the layout-generic kernel
    if ((p.Hkv > 1 && !p.m_hkv) || (p.G > 1 && !p.m_G) || (p.n_splits > 1 && !p.m_splits)) return HQMQ_OK;
    // the outlier variants keep Q and the selector rows behind a smaller V slot
    if (flags && (p.Kc.K > kFlagsTabMax || p.Vc.K > kFlagsTabMax)) return HQMQ_OK;
    // tables are read two codewords (16 bytes) at a time
    if ((p.Kc.K & 1) || (p.Vc.K & 1) || (p.Kc.jsh & 7) || (p.Vc.jsh & 7) || (((uintptr_t)p.Kc.joint | (uintptr_t)p.Vc.joint) & 15))
        return HQMQ_OK;
    *handled = true;
    // long ranges per block (large batches): twelve wavefronts per block, three per SIMD, stream 3-12 % faster; the
    // variants that need more than 168 registers and short launches stay at eight
    const bool wide = (CPL == 8 ? !flags : flags) && p.Tkv / p.n_splits >= 6144;
    // chunked prefill (more than 16 columns per KV head) of plain caches: two column groups per wavefront
    // (only while a block per CU is left: fewer, larger blocks lose more than the shared decode wins)
    const bool two = !flags && p.n_cg > 1 && (int64_t)p.n_splits * ((p.n_cg + 1) / 2) * p.B * p.Hkv >= 256;
    // tables of e4m3 numbers kept as float8 in LDS, on request (decode shapes of the 16-bit layouts at d_h 128)
    if (p.tab_fp8 && CPL == 8 && !two) {
        if (mb == 16 && p.aux_bits == 0 && p.idx_bits == 12) return launch_one<8, 16, 0, 12, DT, kFastWaves, 1, true>(p, flags, grid, st, tm);
        if (mb == 16 && p.aux_bits == 3 && p.idx_bits == 13 && p.Kc.K <= 4608) return launch_one<8, 16, 3, 13, DT, kFastWaves, 1, true>(p, flags, grid, st, tm);
    }
    // plain 16+0 caches with small tables at d_h 128, one column group, eight wavefronts: every load lands in LDS
    if constexpr (CPL == 8) {
        if (mb == 16 && p.aux_bits == 0 && !flags && !two && !wide && !p.no_lds_landing && p.Kc.K <= 2304 && p.Vc.K <= 2304 && p.Kc.K >= 2 &&
            p.Vc.K >= 2 && ((((uintptr_t)p.Q) | (uintptr_t)(p.qsb * 2) | (uintptr_t)(p.qsh * 2) | (uintptr_t)(p.qst * 2)) & 15) == 0)
            return p.idx_bits == 12 ? launch_lds<DT, 12>(p, grid, st, tm) : launch_lds<DT, 0>(p, grid, st, tm);
    }
    if (mb == 16 && p.aux_bits == 0 && p.idx_bits == 12) {
        if (two) return launch_one<CPL, 16, 0, 12, DT, kFastWaves, 2>(p, flags, grid, st, tm);
        return wide ? launch_one<CPL, 16, 0, 12, DT, 12>(p, flags, grid, st, tm) : launch_one<CPL, 16, 0, 12, DT>(p, flags, grid, st, tm);
    }
    if (mb == 16 && p.aux_bits == 0) {
        if (two) return launch_one<CPL, 16, 0, 0, DT, kFastWaves, 2>(p, flags, grid, st, tm);
        return wide ? launch_one<CPL, 16, 0, 0, DT, 12>(p, flags, grid, st, tm) : launch_one<CPL, 16, 0, 0, DT>(p, flags, grid, st, tm);
    }
    if (mb == 12 && p.aux_bits == 1 && CPL == 8 && p.idx_bits == 10 && p.Kc.K <= 1024) {
        if (two) return launch_one<8, 12, 1, 10, DT, kFastWaves, 2>(p, flags, grid, st, tm);
        return wide ? launch_one<8, 12, 1, 10, DT, 12>(p, flags, grid, st, tm) : launch_one<8, 12, 1, 10, DT>(p, flags, grid, st, tm);
    }
    if (mb == 12 && p.aux_bits == 1 && CPL == 8) return launch_one<8, 12, 1, 0, DT>(p, flags, grid, st, tm);
    // (the 16+3 decode needs 182 registers: at three wavefronts per SIMD it spills and runs 40 % slower)
    if (mb == 16 && p.aux_bits == 3 && CPL == 8 && p.idx_bits == 13 && p.Kc.K <= 4608)
        return two ? launch_one<8, 16, 3, 13, DT, kFastWaves, 2>(p, flags, grid, st, tm) : launch_one<8, 16, 3, 13, DT>(p, flags, grid, st, tm);
    if (mb == 16 && p.aux_bits == 3 && CPL == 8) return launch_one<8, 16, 3, 0, DT>(p, flags, grid, st, tm);
    // 16 + 1 bits (s192 with four radius bits, the shape of the reference's published prefill figure): generic field decode
    if (mb == 16 && p.aux_bits == 1 && CPL == 8)
        return two ? launch_one<8, 16, 1, 0, DT, kFastWaves, 2>(p, flags, grid, st, tm) : launch_one<8, 16, 1, 0, DT>(p, flags, grid, st, tm);
    // the remaining widths the layout rule produces for d_h 128 (16 + 2: s96_r6, s192_r5; 12 + 2: s24_r4; 12 + 3: s96_r3,
    // s24_r5), generic field decode: five times faster than the layout-generic kernel at batch 8
    if constexpr (CPL == 8) {
        if (mb == 16 && p.aux_bits == 2)
            return two ? launch_one<8, 16, 2, 0, DT, kFastWaves, 2>(p, flags, grid, st, tm) : launch_one<8, 16, 2, 0, DT>(p, flags, grid, st, tm);
        if (mb == 12 && p.aux_bits == 2)
            return two ? launch_one<8, 12, 2, 0, DT, kFastWaves, 2>(p, flags, grid, st, tm) : launch_one<8, 12, 2, 0, DT>(p, flags, grid, st, tm);
        if (mb == 12 && p.aux_bits == 3)
            return two ? launch_one<8, 12, 3, 0, DT, kFastWaves, 2>(p, flags, grid, st, tm) : launch_one<8, 12, 3, 0, DT>(p, flags, grid, st, tm);
    }
    *handled = false;
    return HQMQ_OK;
}

#ifdef HQMQ_STAMPS
extern "C" int hqmq_debug_set_stamps(void *ptr) { return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_stamps), &ptr, sizeof(ptr)); }
#endif

int launch_attn_fast(const AttnParams &p, int main_bits, bool flags, dim3 grid, size_t table_bytes, hipStream_t st,
                     const LaunchTiming &tm, bool *handled) {
    (void)table_bytes;
    *handled = false;
    if (p.dtype != HQMQ_F16 && p.dtype != HQMQ_BF16) return HQMQ_OK;
    // The kernels of this file form P * (V scale) and convert verbatim chunks in fp16: a bf16 cache whose scales reach
    // 2^15 (the caller says so: wide_range) takes the layout-generic kernel, which carries the range guard.
    if (p.wide_range) return HQMQ_OK;
    if (p.n != 16 && p.n != 32) return HQMQ_OK;
    if (p.t_cap % kSuper) return HQMQ_OK;
    // vector loads of plane rows: main rows 16-byte aligned (checked by the caller), aux and flag rows to their width
    if (p.aux_bits && (((uintptr_t)p.Kc.aux_plane | (uintptr_t)p.Vc.aux_plane) & 3)) return HQMQ_OK;
    if (flags && (!p.Kc.sb_coord || !p.Kc.sb_count || !p.Vc.sb_coord || !p.Vc.sb_count || p.Kc.sb_cap < 2 || p.Vc.sb_cap < 2 || p.Kc.sb_cap >= (1 << 28) || p.Vc.sb_cap >= (1 << 28)))
        return HQMQ_OK;     // the K side walks the entry list
    // 8-byte vector loads of Q rows, table rows and sideband chunks; strides were checked by the caller
    if (p.n == 32) {
        if (p.dtype == HQMQ_F16) return launch_layout<8, HQMQ_F16>(p, main_bits, flags, grid, st, tm, handled);
        return launch_layout<8, HQMQ_BF16>(p, main_bits, flags, grid, st, tm, handled);
    }
    if (p.dtype == HQMQ_F16) return launch_layout<4, HQMQ_F16>(p, main_bits, flags, grid, st, tm, handled);
    return launch_layout<4, HQMQ_BF16>(p, main_bits, flags, grid, st, tm, handled);
}

}  // namespace hqmq
