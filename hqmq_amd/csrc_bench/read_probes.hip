// Measurement kernels (libhqmq_bench.so, built beside the product library and loaded only by bench.py and
// hqmq_amd/bench_ceiling.py): kernels that only READ memory, in the shapes the decode-attention kernels read it.
// What they take is what the memory system allows a launch of that shape; the attention kernel's distance from it is
// what its own arithmetic, tables and merge cost.
//   hqmq_bench_read_planes   the grid, per-wavefront half-steps and per-lane loads of the register-tile attention kernel
//                            (16-byte loads of the main rows of K and V, 8-byte loads of four scales, 32 tokens per step,
//                            a ring of `depth` steps of which depth - 1 are in flight); 16+0 layout at d_h 128
//   hqmq_bench_read_plain    a contiguous buffer, `blocks` x `threads`, `inflight` 16-byte loads per thread outstanding
//   hqmq_bench_read_lds      the same buffer through global_load_lds (memory to LDS without registers): every wavefront
//                            requests its whole share at once, or `ahead` 4 KB pieces ahead of the one it waits for
//   hqmq_bench_empty         a kernel that does nothing: the floor of the event interval
// Every entry point takes two optional hipEvent_t that receive the GPU timestamps of the begin and the end of the dispatch.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

namespace {

constexpr int kSuper = 64;

struct StepWords {
    uint4 k[2], v[2];
    uint2 ks[2], vs[2];
};

template <int DEPTH, int WV>
__global__ __launch_bounds__(WV * 64) void read_planes_kernel(const uint8_t *kmain, const uint8_t *vmain, const uint16_t *kscale,
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
    constexpr int STRIDE = 32 * WV;         // half-steps round-robin over the block's wavefronts
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

template <int U, int NT>
__global__ __launch_bounds__(NT) void read_plain_kernel(const uint4 *__restrict__ p, size_t n, uint32_t *sink) {
    uint32_t acc = 0;
    // every block reads a contiguous share; inside it U loads of consecutive 16 B x NT stretches are in flight
    const size_t per_block = (n + gridDim.x - 1) / gridDim.x;
    const size_t b0 = (size_t)blockIdx.x * per_block, b1 = b0 + per_block < n ? b0 + per_block : n;
    for (size_t i = b0 + threadIdx.x; i < b1; i += (size_t)NT * U) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t j = i + (size_t)u * NT;
            v[u] = p[j < b1 ? j : b1 - 1];
        }
#pragma unroll
        for (int u = 0; u < U; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345u) sink[0] = acc;
}

extern __shared__ uint32_t probe_lds[];
// 512 threads; every wavefront moves `pieces` 4 KB pieces of its block's share to LDS (a ring of 8 pieces of LDS per
// wavefront) and waits for piece i when `ahead` later pieces have been requested (ahead >= pieces: everything at once)
__global__ __launch_bounds__(512) void read_lds_kernel(const uint8_t *__restrict__ p, int pieces, int ahead, uint32_t *sink) {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint8_t *base = p + ((size_t)blockIdx.x * 8 + wave) * (size_t)pieces * 4096;
    const uint32_t voff = lane * 16;
    auto request = [&](int i) {
        const uint64_t sp = (uint64_t)(base + (size_t)i * 4096);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)sp), hi = __builtin_amdgcn_readfirstlane((uint32_t)(sp >> 32));
        const uint8_t *src = (const uint8_t *)(((uint64_t)hi << 32) | lo);
        const uint32_t dst = __builtin_amdgcn_readfirstlane((wave * 4 + (uint32_t)(i & 3)) * 4096u);
        asm volatile("s_mov_b32 m0, %0\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:0\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:1024\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:2048\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:3072"
                     ::"s"(dst), "v"(voff), "s"(src) : "memory");
    };
    uint32_t acc = 0;
    if (ahead >= pieces) {
        for (int i = 0; i < pieces; i++) request(i);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        acc = probe_lds[wave * 4096 + lane];
    } else {            // ahead in {1, 2, 3}: a ring
        for (int i = 0; i < ahead && i < pieces; i++) request(i);
        for (int i = 0; i < pieces; i++) {
            const int later = min(pieces - i - 1, ahead - 1);
            if (later >= 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else if (later == 1) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            acc ^= probe_lds[(wave * 4 + (i & 3)) * 1024 + lane];
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(acc)::"memory");
            if (i + ahead < pieces) request(i + ahead);
        }
    }
    if (acc == 0x12345u) sink[0] = acc;
}

__global__ void empty_kernel(uint32_t *sink) {
    if (sink == (uint32_t *)1) sink[0] = 0;
}

template <class K, class... A>
int launch(K kern, dim3 grid, dim3 block, size_t shmem, void *stream, void *ev0, void *ev1, A... args) {
    if (ev0 || ev1) hipExtLaunchKernelGGL(kern, grid, block, shmem, (hipStream_t)stream, (hipEvent_t)ev0, (hipEvent_t)ev1, 0, args...);
    else hipLaunchKernelGGL(kern, grid, block, shmem, (hipStream_t)stream, args...);
    return (int)hipGetLastError();
}

template <int DEPTH>
int planes_depth(int waves, dim3 grid, void *st, void *e0, void *e1, const uint8_t *km, const uint8_t *vm, const uint16_t *ks,
                 const uint16_t *vs, int64_t t_cap, int Tkv, int n_splits, int nbh, int remap, uint32_t *sink) {
    if (waves == 12) return launch(read_planes_kernel<DEPTH, 12>, grid, dim3(768), 0, st, e0, e1, km, vm, ks, vs, t_cap, Tkv, n_splits, nbh, remap, sink);
    return launch(read_planes_kernel<DEPTH, 8>, grid, dim3(512), 0, st, e0, e1, km, vm, ks, vs, t_cap, Tkv, n_splits, nbh, remap, sink);
}

}  // namespace

extern "C" int64_t hqmq_bench_read_planes_sink_bytes(int nbh, int n_splits) { return (int64_t)nbh * n_splits * 768 * 4; }

// K / V main planes [nbh][t_cap][64 bytes] and scale planes [nbh][t_cap] (16-bit); returns a hipError_t, or -1 for bad arguments
extern "C" int hqmq_bench_read_planes(const void *kmain, const void *vmain, const void *kscale, const void *vscale, int64_t t_cap, int T_kv,
                                      int nbh, int n_splits, int depth, int waves, void *sink, int64_t sink_bytes, void *ev0, void *ev1,
                                      void *stream) {
    if (!kmain || !vmain || !kscale || !vscale || !sink || nbh < 1 || nbh > 65535 || n_splits < 1 || T_kv < 1 || t_cap < T_kv || (t_cap % kSuper))
        return -1;
    if ((waves != 8 && waves != 12) || sink_bytes < hqmq_bench_read_planes_sink_bytes(nbh, n_splits)) return -1;
    dim3 grid((unsigned)n_splits, 1, (unsigned)nbh);
    const int remap = (nbh % 8) == 0;
    const uint8_t *km = (const uint8_t *)kmain, *vm = (const uint8_t *)vmain;
    const uint16_t *ks = (const uint16_t *)kscale, *vs = (const uint16_t *)vscale;
    switch (depth) {
        case 2: return planes_depth<2>(waves, grid, stream, ev0, ev1, km, vm, ks, vs, t_cap, T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        case 3: return planes_depth<3>(waves, grid, stream, ev0, ev1, km, vm, ks, vs, t_cap, T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        case 4: return planes_depth<4>(waves, grid, stream, ev0, ev1, km, vm, ks, vs, t_cap, T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        case 6: return planes_depth<6>(waves, grid, stream, ev0, ev1, km, vm, ks, vs, t_cap, T_kv, n_splits, nbh, remap, (uint32_t *)sink);
        default: return -1;
    }
}

extern "C" int hqmq_bench_read_plain(const void *buf, int64_t bytes, int blocks, int threads, int inflight, void *sink, void *ev0, void *ev1,
                                     void *stream) {
    if (!buf || !sink || bytes < 16 || blocks < 1) return -1;
    const uint4 *p = (const uint4 *)buf;
    const size_t n = (size_t)bytes / 16;
    uint32_t *s = (uint32_t *)sink;
#define HQMQ_PLAIN(U, NT) \
    if (inflight == U && threads == NT) return launch(read_plain_kernel<U, NT>, dim3((unsigned)blocks), dim3(NT), 0, stream, ev0, ev1, p, n, s);
    HQMQ_PLAIN(2, 256) HQMQ_PLAIN(4, 256) HQMQ_PLAIN(8, 256) HQMQ_PLAIN(2, 512) HQMQ_PLAIN(4, 512) HQMQ_PLAIN(8, 512)
#undef HQMQ_PLAIN
    return -1;
}

// `blocks` blocks of 512 threads, every wavefront `pieces` pieces of 4 KB: blocks * 8 * pieces * 4096 bytes are read
extern "C" int hqmq_bench_read_lds(const void *buf, int blocks, int pieces, int ahead, void *sink, void *ev0, void *ev1, void *stream) {
    if (!buf || !sink || blocks < 1 || pieces < 1 || ahead < 1) return -1;
    const size_t shmem = 8 * 4 * 4096;
    static bool once = false;
    if (!once) {
        hipError_t e = hipFuncSetAttribute((const void *)read_lds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
        once = true;
    }
    if (ahead < pieces && ahead > 3) ahead = 3;
    return launch(read_lds_kernel, dim3((unsigned)blocks), dim3(512), shmem, stream, ev0, ev1, (const uint8_t *)buf, pieces, ahead, (uint32_t *)sink);
}

extern "C" int hqmq_bench_empty(int blocks, int threads, void *ev0, void *ev1, void *stream) {
    if (blocks < 1 || threads < 64 || threads > 1024) return -1;
    return launch(empty_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), 0, stream, ev0, ev1, (uint32_t *)nullptr);
}
