// Med3x outlier statistics and sideband compaction.
//
// hqmq_med3x_threshold follows the torch.quantile half of
// OutlierAwareHQMQQuantizer._qdq (src/quantizers/outlier_aware.py:60-69 of the
// reference): per head, the median over every chunk norm of the call (fp32
// interpolation between the two middle order statistics), times the
// multiplier, rounded to D.  The order statistics come from an exact radix
// select: chunk norms are non-negative, so their bit patterns sort like the
// values; 16-bit dtypes need one 32768-bin histogram per head, fp32 a second
// pass over the low 16 bits of the bin(s) holding the two ranks.
//
// hqmq_outlier_compact has no counterpart in the reference: it copies the
// flagged chunks into the fp16/bf16/fp32 sideband in (token, chunk) order.
//
// Compiled with -ffp-contract=off.
#include "common.h"

namespace hqmq {

constexpr int kBins1 = 32768;
constexpr int kBins2 = 65536;
constexpr int kState = 16;  // ints per head

// workspace (uint32 units): hist1[H][kBins1] | state[H][kState] | (fp32 only) hist2[H][2][kBins2]
// state: 0 nan count, 1 key_lo, 2 key_hi, 3 rank_lo within bin, 4 rank_hi within bin
__host__ __device__ inline int64_t ws_words(int H, bool f32) {
    return (int64_t)H * (kBins1 + kState) + (f32 ? (int64_t)H * 2 * kBins2 : 0);
}

__global__ void fill_zero_kernel(uint32_t *p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

template <class D>
__device__ __forceinline__ float chunk_norm(const typename D::storage *xp) {
    return D::rnd(norm4(D::load(xp), D::load(xp + 1), D::load(xp + 2), D::load(xp + 3)));
}

template <class D>
__device__ __forceinline__ uint32_t norm_bits(float nrm) {
    if (D::code == HQMQ_F32) return __float_as_uint(nrm);
    if (D::code == HQMQ_F16) return (uint32_t)__half_as_ushort(__float2half_rn(nrm)) << 16;
    return __float_as_uint(nrm);  // bf16 value: low 16 bits are zero
}

// LEVEL 0: histogram of the top 16 bits. LEVEL 1 (fp32): low 16 bits of norms whose top bits match a selected bin.
template <class D, int LEVEL>
__global__ void med_hist_kernel(const typename D::storage *x, int64_t xsb, int64_t xsh, int64_t xst, int B, int H, int T, int n,
                                uint32_t *ws) {
    const int h = blockIdx.y;
    uint32_t *hist1 = ws + (size_t)h * kBins1;
    uint32_t *state = ws + (size_t)H * kBins1 + (size_t)h * kState;
    uint32_t *hist2 = ws + (size_t)H * (kBins1 + kState) + (size_t)h * 2 * kBins2;
    const int64_t per_head = (int64_t)B * T * n;
    uint32_t key_lo = 0, key_hi = 0;
    if (LEVEL == 1) { key_lo = state[1]; key_hi = state[2]; }
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < per_head; g += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(g % n);
        const int64_t bt = g / n;
        const int t = (int)(bt % T), b = (int)(bt / T);
        const float nrm = chunk_norm<D>(x + b * xsb + h * xsh + (int64_t)t * xst + c * 4);
        if (is_nan(nrm)) {
            if (LEVEL == 0) atomicAdd(&state[0], 1u);
            continue;
        }
        const uint32_t bits = norm_bits<D>(nrm);
        if (LEVEL == 0) atomicAdd(&hist1[bits >> 16], 1u);
        else {
            if ((bits >> 16) == key_lo) atomicAdd(&hist2[bits & 0xffffu], 1u);
            if ((bits >> 16) == key_hi && key_hi != key_lo) atomicAdd(&hist2[kBins2 + (bits & 0xffffu)], 1u);
        }
    }
}

// LEVEL 0 for large calls: the 32768 bins live in LDS (128 KB, one block per CU); a block adds only its non-zero
// bins to the global histogram, a few thousand atomics instead of one per chunk.
template <class D>
__global__ __launch_bounds__(1024) void med_hist_lds_kernel(const typename D::storage *x, int64_t xsb, int64_t xsh, int64_t xst, int B,
                                                            int H, int T, int n, uint32_t *ws) {
    extern __shared__ uint32_t lh[];    // [kBins1] + 1 (NaN count)
    const int h = blockIdx.y;
    uint32_t *hist1 = ws + (size_t)h * kBins1;
    uint32_t *state = ws + (size_t)H * kBins1 + (size_t)h * kState;
    for (int i = threadIdx.x; i <= kBins1; i += 1024) lh[i] = 0;
    __syncthreads();
    const int64_t per_head = (int64_t)B * T * n;
    for (int64_t g = (int64_t)blockIdx.x * 1024 + threadIdx.x; g < per_head; g += (int64_t)gridDim.x * 1024) {
        int c, t, b;
        if (per_head < 0x7fffffff) {
            const uint32_t g32 = (uint32_t)g, bt = g32 / (uint32_t)n;
            c = (int)(g32 - bt * (uint32_t)n);
            b = (int)(bt / (uint32_t)T);
            t = (int)(bt - (uint32_t)b * (uint32_t)T);
        } else {
            c = (int)(g % n);
            const int64_t bt = g / n;
            t = (int)(bt % T);
            b = (int)(bt / T);
        }
        const float nrm = chunk_norm<D>(x + b * xsb + h * xsh + (int64_t)t * xst + c * 4);
        if (is_nan(nrm)) atomicAdd(&lh[kBins1], 1u);
        else atomicAdd(&lh[norm_bits<D>(nrm) >> 16], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kBins1; i += 1024) {
        const uint32_t v = lh[i];
        if (v) atomicAdd(&hist1[i], v);
    }
    if (threadIdx.x == 0 && lh[kBins1]) atomicAdd(&state[0], lh[kBins1]);
}

// Finds the bins holding 0-based ranks r_lo <= r_hi in a histogram of `bins` counters.
// One block of 1024 threads: every thread sums its bins/1024 consecutive counters, a block-wide scan gives each
// thread the rank range of its segment, and the thread whose range holds a wanted rank walks its own segment.
__device__ void select_two(const uint32_t *hist, int bins, int64_t r_lo, int64_t r_hi, uint32_t *key_lo, uint32_t *key_hi,
                           int64_t *in_lo, int64_t *in_hi) {
    __shared__ unsigned long long part[1024];
    __shared__ uint32_t res[2];
    __shared__ long long resr[2];
    const int per = bins / 1024;
    unsigned long long s = 0;
    for (int i = 0; i < per; i++) s += hist[threadIdx.x * per + i];
    part[threadIdx.x] = s;
    if (threadIdx.x < 2) { res[threadIdx.x] = (uint32_t)(bins - 1); resr[threadIdx.x] = 0; }
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {  // inclusive Hillis-Steele scan
        const unsigned long long v = (int)threadIdx.x >= off ? part[threadIdx.x - off] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    const unsigned long long incl = part[threadIdx.x], excl = incl - s;
    const int64_t want[2] = {r_lo, r_hi};
    for (int which = 0; which < 2; which++) {
        const unsigned long long w = (unsigned long long)want[which];
        if (w >= excl && w < incl) {
            unsigned long long r2 = excl;
            for (int j = 0; j < per; j++) {
                const uint32_t cnt = hist[threadIdx.x * per + j];
                if (w < r2 + cnt) {
                    res[which] = (uint32_t)(threadIdx.x * per + j);
                    resr[which] = (long long)(w - r2);
                    break;
                }
                r2 += cnt;
            }
        }
    }
    __syncthreads();
    *key_lo = res[0]; *key_hi = res[1];
    *in_lo = resr[0]; *in_hi = resr[1];
    __syncthreads();
}

template <class D>
__device__ __forceinline__ void finish_threshold(float a, float b, bool same, float mult, int h, float *median,
                                                 typename D::storage *thr) {
    float med;
    if (same) med = a;
    else {
        const float d = b - a;
        const float e = d * 0.5f;
        med = b - e;
    }
    median[h] = med;
    const float t32 = med * mult;
    D::store(thr + h, D::rnd(t32));
}

template <class D>
__global__ __launch_bounds__(1024) void med_select1_kernel(uint32_t *ws, int H, int64_t per_head, float mult, float *median,
                                                           typename D::storage *thr, int32_t *n_out) {
    const int h = blockIdx.x;
    const uint32_t *hist1 = ws + (size_t)h * kBins1;
    uint32_t *state = ws + (size_t)H * kBins1 + (size_t)h * kState;
    if (state[0] > 0) {  // a NaN norm makes the quantile NaN, the mask empty
        if (threadIdx.x == 0) {
            median[h] = NAN;
            D::store(thr + h, NAN);
            if (n_out) n_out[h] = 0;
            state[1] = 0xffffffffu; state[2] = 0xffffffffu;
        }
        return;
    }
    uint32_t klo, khi;
    int64_t ilo, ihi;
    select_two(hist1, kBins1, (per_head - 1) / 2, per_head / 2, &klo, &khi, &ilo, &ihi);
    if (D::code == HQMQ_F32) {
        if (threadIdx.x == 0) { state[1] = klo; state[2] = khi; state[3] = (uint32_t)ilo; state[4] = (uint32_t)ihi; }
        return;
    }
    __shared__ float thr_sh;
    if (threadIdx.x == 0) {
        const float a = (D::code == HQMQ_F16) ? __half2float(__ushort_as_half((uint16_t)klo)) : __uint_as_float(klo << 16);
        const float b = (D::code == HQMQ_F16) ? __half2float(__ushort_as_half((uint16_t)khi)) : __uint_as_float(khi << 16);
        finish_threshold<D>(a, b, (per_head - 1) / 2 == per_head / 2, mult, h, median, thr);
        thr_sh = D::load(thr + h);
    }
    __syncthreads();
    if (n_out) {  // chunks with norm > thr: bins above the threshold's own bin
        __shared__ unsigned long long cnt_sh;
        if (threadIdx.x == 0) cnt_sh = 0;
        __syncthreads();
        const float tv = thr_sh;
        unsigned long long s = 0;
        for (int k = threadIdx.x; k < kBins1; k += blockDim.x) {
            const float v = (D::code == HQMQ_F16) ? __half2float(__ushort_as_half((uint16_t)k)) : __uint_as_float((uint32_t)k << 16);
            if (v > tv) s += hist1[k];
        }
        atomicAdd(&cnt_sh, s);
        __syncthreads();
        if (threadIdx.x == 0) n_out[h] = (int32_t)cnt_sh;
    }
}

// Small calls (a decode step appends B * n chunks per head): norms, exact radix select and count in one launch,
// one block per head, the 16-bit keys in LDS.  16-bit dtypes only.
constexpr int kSmallMax = 8192;

// rank -> (bin holding it, rank inside the bin) over the 256 counters of `hist`; every thread of the block calls it
__device__ __forceinline__ void find_bin256(const uint32_t *hist, uint32_t rank, uint32_t *wave_tot, uint32_t *res,
                                            uint32_t &bin, uint32_t &inner) {
    const int tid = threadIdx.x;
    uint32_t v = 0, incl = 0;
    if (tid < 256) {
        v = hist[tid];
        incl = v;
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t u = __shfl_up(incl, o, 64);
            if ((tid & 63) >= o) incl += u;
        }
        if ((tid & 63) == 63) wave_tot[tid >> 6] = incl;
    }
    __syncthreads();
    if (tid < 256) {
        for (int w = 0; w < (tid >> 6); w++) incl += wave_tot[w];
        const uint32_t excl = incl - v;
        if (rank >= excl && rank < incl) { res[0] = (uint32_t)tid; res[1] = rank - excl; }
    }
    __syncthreads();
    bin = res[0];
    inner = res[1];
    __syncthreads();
}

struct MedSmall {
    const void *x; int64_t xsb, xsh, xst;
    int B, T, n;
    float mult;
    float *median; void *thr; int32_t *n_out;
};

// NT threads (at least 256)
template <class D, int NT>
__device__ __forceinline__ void med_small_body(const MedSmall &a) {
    const typename D::storage *x = (const typename D::storage *)a.x;
    typename D::storage *thr = (typename D::storage *)a.thr;
    const int64_t xsb = a.xsb, xsh = a.xsh, xst = a.xst;
    const int B = a.B, T = a.T, n = a.n;
    const float mult = a.mult;
    float *median = a.median;
    int32_t *n_out = a.n_out;
    __shared__ uint16_t keys[kSmallMax];
    __shared__ uint32_t hist[256], wave_tot[4], res[2], nan_count, gt_count;
    __shared__ float thr_sh;
    const int h = blockIdx.x, tid = threadIdx.x;
    const int per_head = B * T * n;
    if (tid == 0) { nan_count = 0; gt_count = 0; res[0] = 255; res[1] = 0; }
    __syncthreads();
    for (int g = tid; g < per_head; g += NT) {
        const int bt = g / n, c = g - bt * n, b = bt / T, t = bt - b * T;
        const float nrm = chunk_norm<D>(x + b * xsb + h * xsh + (int64_t)t * xst + c * 4);
        if (is_nan(nrm)) { atomicAdd(&nan_count, 1u); keys[g] = 0xffffu; }
        else keys[g] = (uint16_t)(norm_bits<D>(nrm) >> 16);
    }
    __syncthreads();
    if (nan_count > 0) {  // a NaN norm makes the quantile NaN, the mask empty
        if (tid == 0) {
            median[h] = NAN;
            D::store(thr + h, NAN);
            if (n_out) n_out[h] = 0;
        }
        return;
    }
    auto select = [&](uint32_t rank) -> uint32_t {
        uint32_t hi, in_hi, lo, in_lo;
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        for (int g = tid; g < per_head; g += NT) atomicAdd(&hist[keys[g] >> 8], 1u);
        __syncthreads();
        find_bin256(hist, rank, wave_tot, res, hi, in_hi);
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        for (int g = tid; g < per_head; g += NT)
            if ((uint32_t)(keys[g] >> 8) == hi) atomicAdd(&hist[keys[g] & 255u], 1u);
        __syncthreads();
        find_bin256(hist, in_hi, wave_tot, res, lo, in_lo);
        return (hi << 8) | lo;
    };
    const uint32_t r_lo = (uint32_t)((per_head - 1) / 2), r_hi = (uint32_t)(per_head / 2);
    const uint32_t klo = select(r_lo);
    const uint32_t khi = r_hi == r_lo ? klo : select(r_hi);
    if (tid == 0) {
        const float a = (D::code == HQMQ_F16) ? __half2float(__ushort_as_half((uint16_t)klo)) : __uint_as_float(klo << 16);
        const float b = (D::code == HQMQ_F16) ? __half2float(__ushort_as_half((uint16_t)khi)) : __uint_as_float(khi << 16);
        finish_threshold<D>(a, b, r_lo == r_hi, mult, h, median, thr);
        thr_sh = D::load(thr + h);
    }
    __syncthreads();
    if (n_out) {
        const float tv = thr_sh;
        uint32_t cnt = 0;
        for (int g = tid; g < per_head; g += NT) {
            const uint32_t k = keys[g];
            const float v = (D::code == HQMQ_F16) ? __half2float(__ushort_as_half((uint16_t)k)) : __uint_as_float(k << 16);
            if (v > tv) cnt++;
        }
        if (cnt) atomicAdd(&gt_count, cnt);
        __syncthreads();
        if (tid == 0) n_out[h] = (int32_t)gt_count;
    }
}

template <class D, int NT>
__global__ __launch_bounds__(NT) void med_small_kernel(MedSmall a) {
    med_small_body<D, NT>(a);
}
// two tensors of equal shape: blockIdx.y picks one
template <class D, int NT>
__global__ __launch_bounds__(NT) void med_small_pair_kernel(MedSmall a, MedSmall b) {
    med_small_body<D, NT>(blockIdx.y ? b : a);
}

__global__ __launch_bounds__(1024) void med_select2_kernel(uint32_t *ws, int H, int64_t per_head, float mult, float *median,
                                                           float *thr) {
    const int h = blockIdx.x;
    uint32_t *state = ws + (size_t)H * kBins1 + (size_t)h * kState;
    const uint32_t *hist2 = ws + (size_t)H * (kBins1 + kState) + (size_t)h * 2 * kBins2;
    if (state[0] > 0) return;
    const uint32_t klo = state[1], khi = state[2];
    uint32_t l0, l1, d0, d1;
    int64_t i0, i1;
    if (klo == khi) {
        select_two(hist2, kBins2, state[3], state[4], &l0, &l1, &i0, &i1);
    } else {
        select_two(hist2, kBins2, state[3], state[3], &l0, &d0, &i0, &i1);
        select_two(hist2 + kBins2, kBins2, state[4], state[4], &l1, &d1, &i0, &i1);
    }
    if (threadIdx.x == 0) {
        const float a = __uint_as_float((klo << 16) | l0), b = __uint_as_float((khi << 16) | l1);
        finish_threshold<F32>(a, b, (per_head - 1) / 2 == per_head / 2, mult, h, median, thr);
    }
}

__global__ void count_gt_kernel(const float *x, int64_t xsb, int64_t xsh, int64_t xst, int B, int T, int n, const float *thr,
                                int32_t *n_out) {
    const int h = blockIdx.y;
    const float tv = thr[h];
    const int64_t per_head = (int64_t)B * T * n;
    int cnt = 0;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < per_head; g += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(g % n);
        const int64_t bt = g / n;
        const int t = (int)(bt % T), b = (int)(bt / T);
        if (chunk_norm<F32>(x + b * xsb + h * xsh + (int64_t)t * xst + c * 4) > tv) cnt++;
    }
    if (cnt) atomicAdd(&n_out[h], cnt);
}

// One block of NT threads per (b, h): walks the T new rows in order, NT rows per step (one wavefront for short
// appends: its barriers cost nothing).
template <class D, int NT>
__device__ __forceinline__ void compact_body(const CompactCall &a) {
    using ST = typename D::storage;
    const ST *x = (const ST *)a.x;
    ST *sideband = (ST *)a.sideband;
    const int64_t xsb = a.xsb, xsh = a.xsh, xst = a.xst, t_cap = a.t_cap, sb_cap = a.sb_cap;
    const int H = a.H, T = a.T, n = a.n, t_off = a.t_off;
    const uint8_t *flag_plane = a.flag_plane;
    const int32_t *pos = a.pos;
    int32_t *sb_tile_off = a.sb_tile_off, *sb_count = a.sb_count, *overflow = a.overflow;
    uint16_t *sb_coord = a.sb_coord;
    __shared__ int scan[NT];
    __shared__ int base_sh;
    const int bh = blockIdx.x, b = bh / H, h = bh - b * H;
    const int frb = (n + 7) >> 3;
    const int64_t row0 = (pos ? pos[b] : 0) + t_off;
    const int64_t tiles = (t_cap + kTile - 1) / kTile;
    if (threadIdx.x == 0) base_sh = sb_count[bh];
    __syncthreads();
    for (int t0 = 0; t0 < T; t0 += NT) {
        const int t = t0 + threadIdx.x;
        const int64_t row = row0 + t;
        const bool live = t < T && row < t_cap;
        int cnt = 0;
        const uint8_t *fr = flag_plane + ((size_t)bh * t_cap + (live ? row : 0)) * frb;
        if (live)
            for (int by = 0; by < frb; by++) cnt += __popc((uint32_t)fr[by]);
        scan[threadIdx.x] = cnt;
        __syncthreads();
        for (int off = 1; off < NT; off <<= 1) {  // inclusive Hillis-Steele scan
            int v = (int)threadIdx.x >= off ? scan[threadIdx.x - off] : 0;
            __syncthreads();
            scan[threadIdx.x] += v;
            __syncthreads();
        }
        const int base = base_sh;
        const int before = base + scan[threadIdx.x] - cnt;
        if (live) {
            if ((row & (kTile - 1)) == 0) sb_tile_off[(size_t)bh * tiles + (row >> 4)] = before;
            int k = before;
            const ST *xr = x + b * xsb + h * xsh + (int64_t)t * xst;
            uint64_t own[4] = {0, 0, 0, 0};                        // the row's flags as they were, in registers (bits may be cleared below)
            if (cnt) {
#pragma unroll
                for (int by = 0; by < 32; by++)
                    if (by < frb) own[by >> 3] |= (uint64_t)fr[by] << (8 * (by & 7));
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                for (uint64_t bits = own[q]; bits; bits &= bits - 1) {
                    const int c = 64 * q + __builtin_ctzll(bits);
                    if (c >= n) break;
                    if (k < sb_cap) {
                        ST *dst = sideband + ((size_t)bh * sb_cap + k) * 4;
                        for (int j = 0; j < 4; j++) dst[j] = xr[c * 4 + j];
                        if (sb_coord) sb_coord[(size_t)bh * sb_cap + k] = (uint16_t)(((row & (kTile - 1)) << 8) | c);
                    } else {
                        *overflow = 1;
                        degrade_to_plain<D>(a, (size_t)bh * t_cap + row, c, xr + c * 4);
                    }
                    k++;
                }
            }
        }
        __syncthreads();
        if (threadIdx.x == NT - 1) base_sh = base + scan[NT - 1];
        __syncthreads();
    }
    if (threadIdx.x == 0) sb_count[bh] = base_sh;
}

template <class D, int NT>
__global__ __launch_bounds__(NT) void compact_kernel(CompactCall a) {
    compact_body<D, NT>(a);
}
// two tensors of equal shape: blockIdx.y picks one
template <class D, int NT>
__global__ __launch_bounds__(NT) void compact_pair_kernel(CompactCall a, CompactCall b) {
    compact_body<D, NT>(blockIdx.y ? b : a);
}

// ---- bulk appends (whole 16-row tiles from an aligned first row): three passes with one thread per tile / row ----
// Pass 1: flagged chunks of every new tile -> sb_tile_off[tile] (a count for now).
__global__ void tile_count_kernel(const uint8_t *flag_plane, int64_t t_cap, int row0, int T, int frb, int n_tiles, int32_t *sb_tile_off) {
    const int bh = blockIdx.y;
    const int64_t tiles = (t_cap + kTile - 1) / kTile;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_tiles) return;
    const int r_begin = row0 + i * kTile, r_end = min(row0 + T, r_begin + kTile);
    const uint8_t *fr = flag_plane + ((size_t)bh * t_cap + r_begin) * frb;
    int cnt = 0;
    for (int k = 0; k < (r_end - r_begin) * frb; k++) cnt += __popc((uint32_t)fr[k]);
    sb_tile_off[(size_t)bh * tiles + (r_begin >> 4)] = cnt;
}
// Pass 2: one block per (b, h): counts -> sideband offsets (exclusive scan behind the chunks already stored).
__global__ __launch_bounds__(1024) void tile_scan_kernel(int64_t t_cap, int row0, int n_tiles, int32_t *sb_tile_off, int32_t *sb_count) {
    __shared__ int part[1024];
    const int bh = blockIdx.x;
    const int64_t tiles = (t_cap + kTile - 1) / kTile;
    int32_t *to = sb_tile_off + (size_t)bh * tiles + (row0 >> 4);
    const int per = (n_tiles + 1023) / 1024;
    const int i0 = threadIdx.x * per, i1 = min(n_tiles, i0 + per);
    int s = 0;
    for (int i = i0; i < i1; i++) s += to[i];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const int v = (int)threadIdx.x >= off ? part[threadIdx.x - off] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    const int base = sb_count[bh];
    int run = base + part[threadIdx.x] - s;
    for (int i = i0; i < i1; i++) {
        const int c = to[i];
        to[i] = run;
        run += c;
    }
    __syncthreads();
    if (threadIdx.x == 1023) sb_count[bh] = base + part[1023];
}
// Pass 3: one thread per new row copies the row's flagged chunks behind those of the tile's earlier rows.
// (A row whose entries do not fit clears flag bits while its neighbours count them: every entry they then fail to
// count lay beyond the capacity, so their own entries still come out beyond it, and the offsets of the entries that
// fit do not move.)
template <class D>
__global__ void tile_copy_kernel(CompactCall a) {
    using ST = typename D::storage;
    const ST *x = (const ST *)a.x;
    ST *sideband = (ST *)a.sideband;
    const int H = a.H, T = a.T, n = a.n, row0 = a.t_off;
    const int64_t t_cap = a.t_cap, sb_cap = a.sb_cap;
    const uint8_t *flag_plane = a.flag_plane;
    const int bh = blockIdx.y, b = bh / H, h = bh - b * H;
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= T) return;
    const int frb = (n + 7) >> 3;
    const int64_t tiles = (t_cap + kTile - 1) / kTile;
    const int row = row0 + t, tile_row = row & ~(kTile - 1);
    const uint8_t *fr = flag_plane + ((size_t)bh * t_cap + row) * frb;
    // the row's flag bits as they are now, in registers (up to 256 chunks): rows whose entries do not fit clear bits
    // while this one runs
    uint64_t mine[4] = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < 32; k++)
        if (k < frb) mine[k >> 3] |= (uint64_t)fr[k] << (8 * (k & 7));
    if (!(mine[0] | mine[1] | mine[2] | mine[3])) return;
    int before = a.sb_tile_off[(size_t)bh * tiles + (row >> 4)];
    const uint8_t *f0 = flag_plane + ((size_t)bh * t_cap + tile_row) * frb;
    for (int k = 0; k < (row - tile_row) * frb; k++) before += __popc((uint32_t)f0[k]);
    const ST *xr = x + b * a.xsb + h * a.xsh + (int64_t)t * a.xst;
    int k = before;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        for (uint64_t bits = mine[q]; bits; bits &= bits - 1) {
            const int c = 64 * q + __builtin_ctzll(bits);
            if (c >= n) break;
            if (k < sb_cap) {
                ST *dst = sideband + ((size_t)bh * sb_cap + k) * 4;
                for (int j = 0; j < 4; j++) dst[j] = xr[c * 4 + j];
                if (a.sb_coord) a.sb_coord[(size_t)bh * sb_cap + k] = (uint16_t)(((row & (kTile - 1)) << 8) | c);
            } else {
                *a.overflow = 1;
                degrade_to_plain<D>(a, (size_t)bh * t_cap + row, c, xr + c * 4);
            }
            k++;
        }
    }
}

}  // namespace hqmq

using namespace hqmq;

extern "C" int64_t hqmq_med3x_workspace_bytes(int H, int dtype) {
    if (H < 1) return 0;
    return ws_words(H, dtype == HQMQ_F32) * 4;
}

template <class D>
static int run_med3x(const void *x, int64_t xsb, int64_t xsh, int64_t xst, int B, int H, int T, int n, float mult, uint32_t *ws,
                     float *median, void *thr, int32_t *n_out, hipStream_t st) {
    using ST = typename D::storage;
    const bool f32 = D::code == HQMQ_F32;
    const int64_t words = ws_words(H, f32);
    const int64_t per_head = (int64_t)B * T * n;
    if (!f32 && per_head <= kSmallMax) {
        const MedSmall a{x, xsb, xsh, xst, B, T, n, mult, median, thr, n_out};
        hipLaunchKernelGGL((med_small_kernel<D, 1024>), dim3(H), dim3(1024), 0, st, a);
        return hip_status(hipGetLastError());
    }
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, st, ws, words);
    int gx = (int)((per_head + 255) / 256);
    if (gx > 2048) gx = 2048;
    if (per_head >= (1 << 18)) {
        const size_t lds = (size_t)(kBins1 + 1) * sizeof(uint32_t);
        hipError_t e = hipFuncSetAttribute((const void *)med_hist_lds_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        int gl = (int)((per_head + 16383) / 16384);
        if (gl > 128) gl = 128;
        hipLaunchKernelGGL(med_hist_lds_kernel<D>, dim3(gl, H), dim3(1024), lds, st, (const ST *)x, xsb, xsh, xst, B, H, T, n, ws);
    } else {
        hipLaunchKernelGGL((med_hist_kernel<D, 0>), dim3(gx, H), dim3(256), 0, st, (const ST *)x, xsb, xsh, xst, B, H, T, n, ws);
    }
    hipLaunchKernelGGL(med_select1_kernel<D>, dim3(H), dim3(1024), 0, st, ws, H, per_head, mult, median, (ST *)thr, n_out);
    if (f32) {
        hipLaunchKernelGGL((med_hist_kernel<D, 1>), dim3(gx, H), dim3(256), 0, st, (const ST *)x, xsb, xsh, xst, B, H, T, n, ws);
        hipLaunchKernelGGL(med_select2_kernel, dim3(H), dim3(1024), 0, st, ws, H, per_head, mult, median, (float *)thr);
        if (n_out) {
            hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, st, (uint32_t *)n_out, (int64_t)H);
            hipLaunchKernelGGL(count_gt_kernel, dim3(gx, H), dim3(256), 0, st, (const float *)x, xsb, xsh, xst, B, T, n,
                               (const float *)thr, n_out);
        }
    }
    return hip_status(hipGetLastError());
}

static int check_med3x(const Med3xCall &c) {
    if (!c.x || !c.ws || !c.median || !c.thr) return HQMQ_ERR_NULL;
    if (c.B < 1 || c.H < 1 || c.H > 65535 || c.T < 1 || c.n < 1) return HQMQ_ERR_SHAPE;
    if (c.dtype != HQMQ_F32 && c.dtype != HQMQ_F16 && c.dtype != HQMQ_BF16) return HQMQ_ERR_DTYPE;
    if (c.ws_bytes < hqmq_med3x_workspace_bytes(c.H, c.dtype)) return HQMQ_ERR_WORKSPACE;
    if (((uintptr_t)c.ws & 3) != 0) return HQMQ_ERR_ALIGN;
    return HQMQ_OK;
}

static int med3x_one(const Med3xCall &c, hipStream_t st) {
    uint32_t *ws = (uint32_t *)c.ws;
    switch (c.dtype) {
        case HQMQ_F32: return run_med3x<F32>(c.x, c.xsb, c.xsh, c.xst, c.B, c.H, c.T, c.n, c.mult, ws, c.median, c.thr, c.n_out, st);
        case HQMQ_F16: return run_med3x<F16>(c.x, c.xsb, c.xsh, c.xst, c.B, c.H, c.T, c.n, c.mult, ws, c.median, c.thr, c.n_out, st);
        default: return run_med3x<BF16>(c.x, c.xsb, c.xsh, c.xst, c.B, c.H, c.T, c.n, c.mult, ws, c.median, c.thr, c.n_out, st);
    }
}

int hqmq::med3x_calls(const Med3xCall *c, int count, hipStream_t st) {
    for (int i = 0; i < count; i++) {
        const int rc = check_med3x(c[i]);
        if (rc) return rc;
    }
    if (count == 2 && c[0].dtype == c[1].dtype && c[0].dtype != HQMQ_F32 && c[0].B == c[1].B && c[0].H == c[1].H &&
        c[0].T == c[1].T && c[0].n == c[1].n && (int64_t)c[0].B * c[0].T * c[0].n <= kSmallMax) {
        const MedSmall a{c[0].x, c[0].xsb, c[0].xsh, c[0].xst, c[0].B, c[0].T, c[0].n, c[0].mult, c[0].median, c[0].thr, c[0].n_out};
        const MedSmall b{c[1].x, c[1].xsb, c[1].xsh, c[1].xst, c[1].B, c[1].T, c[1].n, c[1].mult, c[1].median, c[1].thr, c[1].n_out};
        const dim3 grid(c[0].H, 2);
        // (256 threads for a few thousand keys measured slower: 11.9 against 8.7 us, the norms load eight deep per thread)
        if (c[0].dtype == HQMQ_F16) hipLaunchKernelGGL((med_small_pair_kernel<F16, 1024>), grid, dim3(1024), 0, st, a, b);
        else hipLaunchKernelGGL((med_small_pair_kernel<BF16, 1024>), grid, dim3(1024), 0, st, a, b);
        return hip_status(hipGetLastError());
    }
    for (int i = 0; i < count; i++) {
        const int rc = med3x_one(c[i], st);
        if (rc) return rc;
    }
    return HQMQ_OK;
}

extern "C" int hqmq_med3x_threshold(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int dtype, int B,
                                    int H, int T, int n_chunks, float mult, void *workspace, int64_t workspace_bytes,
                                    float *median, void *thr, int32_t *n_out, void *stream) {
    const Med3xCall c{x, x_stride_b, x_stride_h, x_stride_t, dtype, B, H, T, n_chunks, mult, workspace, workspace_bytes,
                      median, thr, n_out};
    return med3x_calls(&c, 1, (hipStream_t)stream);
}

int hqmq::check_compact(const CompactCall &c) {
    if (!c.x || !c.flag_plane || !c.sideband || !c.sb_tile_off || !c.sb_count || !c.overflow) return HQMQ_ERR_NULL;
    if (c.B < 1 || c.H < 1 || c.T < 0 || c.n < 1 || c.t_cap < 1 || c.sb_cap < 1 || c.t_off < 0) return HQMQ_ERR_SHAPE;
    if (c.dtype != HQMQ_F32 && c.dtype != HQMQ_F16 && c.dtype != HQMQ_BF16) return HQMQ_ERR_DTYPE;
    return HQMQ_OK;
}

// whole 16-row tiles from an aligned first row: the three tile-parallel passes
static bool bulk_compact(const CompactCall &c) {
    return !c.pos && (c.t_off % kTile) == 0 && c.T >= 512 && (int64_t)c.t_off + c.T <= c.t_cap && c.B * c.H <= 65535;
}

static int compact_one(const CompactCall &c, hipStream_t st) {
    if (c.T == 0) return HQMQ_OK;
    if (bulk_compact(c)) {
        const int n_tiles = (c.T + kTile - 1) / kTile, frb = (c.n + 7) >> 3;
        hipLaunchKernelGGL(tile_count_kernel, dim3((n_tiles + 255) / 256, c.B * c.H), dim3(256), 0, st, c.flag_plane, c.t_cap, c.t_off,
                           c.T, frb, n_tiles, c.sb_tile_off);
        hipLaunchKernelGGL(tile_scan_kernel, dim3(c.B * c.H), dim3(1024), 0, st, c.t_cap, c.t_off, n_tiles, c.sb_tile_off, c.sb_count);
        dim3 cgrid((c.T + 255) / 256, c.B * c.H);
#define COPY(DT) hipLaunchKernelGGL(tile_copy_kernel<DT>, cgrid, dim3(256), 0, st, c)
        switch (c.dtype) {
            case HQMQ_F32: COPY(F32); break;
            case HQMQ_F16: COPY(F16); break;
            default: COPY(BF16); break;
        }
#undef COPY
        return hip_status(hipGetLastError());
    }
    dim3 grid(c.B * c.H);
#define LAUNCH(NT)                                                                                              \
    switch (c.dtype) {                                                                                          \
        case HQMQ_F32: hipLaunchKernelGGL((compact_kernel<F32, NT>), grid, dim3(NT), 0, st, c); break;          \
        case HQMQ_F16: hipLaunchKernelGGL((compact_kernel<F16, NT>), grid, dim3(NT), 0, st, c); break;          \
        default: hipLaunchKernelGGL((compact_kernel<BF16, NT>), grid, dim3(NT), 0, st, c); break;               \
    }
    if (c.T <= 64) { LAUNCH(64) } else { LAUNCH(1024) }
#undef LAUNCH
    return hip_status(hipGetLastError());
}

int hqmq::compact_calls(const CompactCall *c, int count, hipStream_t st) {
    for (int i = 0; i < count; i++) {
        const int rc = check_compact(c[i]);
        if (rc) return rc;
    }
    if (count == 2 && c[0].T > 0 && c[0].dtype == c[1].dtype && c[0].B == c[1].B && c[0].H == c[1].H && c[0].T == c[1].T &&
        c[0].n == c[1].n && !bulk_compact(c[0]) && !bulk_compact(c[1])) {
        dim3 grid(c[0].B * c[0].H, 2);
#define LAUNCH(NT)                                                                                                         \
    switch (c[0].dtype) {                                                                                                  \
        case HQMQ_F32: hipLaunchKernelGGL((compact_pair_kernel<F32, NT>), grid, dim3(NT), 0, st, c[0], c[1]); break;       \
        case HQMQ_F16: hipLaunchKernelGGL((compact_pair_kernel<F16, NT>), grid, dim3(NT), 0, st, c[0], c[1]); break;       \
        default: hipLaunchKernelGGL((compact_pair_kernel<BF16, NT>), grid, dim3(NT), 0, st, c[0], c[1]); break;            \
    }
        if (c[0].T <= 64) { LAUNCH(64) } else { LAUNCH(1024) }
#undef LAUNCH
        return hip_status(hipGetLastError());
    }
    for (int i = 0; i < count; i++) {
        const int rc = compact_one(c[i], st);
        if (rc) return rc;
    }
    return HQMQ_OK;
}

extern "C" int hqmq_outlier_compact(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int dtype, int B,
                                    int H, int T, int n_chunks, uint8_t *flag_plane, int64_t t_cap, int t_off,
                                    const int32_t *pos, void *sideband, int64_t sb_cap, int32_t *sb_tile_off,
                                    int32_t *sb_count, int32_t *overflow, uint16_t *sb_coord, const hqmq_packed_rows *planes,
                                    void *stream) {
    CompactCall c{x, x_stride_b, x_stride_h, x_stride_t, dtype, B, H, T, n_chunks, flag_plane, t_cap, t_off, pos,
                  sideband, sb_cap, sb_tile_off, sb_count, overflow, sb_coord, nullptr, nullptr, nullptr, 0, 0, 0, 0};
    if (planes) {
        if (!planes->main_plane || !planes->scale_plane || (planes->aux_bits > 0 && !planes->aux_plane)) return HQMQ_ERR_NULL;
        if (planes->idx_bits < 1 || planes->main_bits < planes->idx_bits - 8 || planes->main_bits > 16 || planes->aux_bits < 0 ||
            planes->aux_bits > 8 || planes->qmax < 1)
            return HQMQ_ERR_LAYOUT;
        c.main_plane = planes->main_plane; c.aux_plane = planes->aux_plane; c.scale_plane = planes->scale_plane;
        c.idx_bits = planes->idx_bits; c.main_bits = planes->main_bits; c.aux_bits = planes->aux_bits; c.qmax = planes->qmax;
    }
    return compact_calls(&c, 1, (hipStream_t)stream);
}

namespace hqmq {
template <class D>
__global__ void outlier_mask_kernel(const typename D::storage *x, int64_t xsb, int64_t xsh, int64_t xst, int B, int H, int T, int n,
                                    const typename D::storage *thr, uint8_t *mask) {
    const int64_t total = (int64_t)B * H * T * n;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(g % n);
        const int64_t row = g / n;
        const int t = (int)(row % T), h = (int)((row / T) % H), b = (int)(row / ((int64_t)T * H));
        mask[g] = chunk_norm<D>(x + b * xsb + h * xsh + (int64_t)t * xst + c * 4) > D::load(thr + h) ? 1 : 0;
    }
}
}  // namespace hqmq

extern "C" int hqmq_outlier_mask(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int dtype, int B,
                                 int H, int T, int n_chunks, const void *thr, uint8_t *mask, void *stream) {
    if (!x || !thr || !mask) return HQMQ_ERR_NULL;
    if (B < 1 || H < 1 || T < 0 || n_chunks < 1) return HQMQ_ERR_SHAPE;
    if (T == 0) return HQMQ_OK;
    const int64_t total = (int64_t)B * H * T * n_chunks;
    int64_t g = (total + 255) / 256;
    if (g > (1 << 20)) g = 1 << 20;
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(DT, ST)                                                                                                      \
    hipLaunchKernelGGL(outlier_mask_kernel<DT>, dim3((unsigned)g), dim3(256), 0, st, (const ST *)x, x_stride_b, x_stride_h, \
                       x_stride_t, B, H, T, n_chunks, (const ST *)thr, mask)
    switch (dtype) {
        case HQMQ_F32: LAUNCH(F32, float); break;
        case HQMQ_F16: LAUNCH(F16, uint16_t); break;
        case HQMQ_BF16: LAUNCH(BF16, uint16_t); break;
        default: return HQMQ_ERR_DTYPE;
    }
#undef LAUNCH
    return hip_status(hipGetLastError());
}
