#!/usr/bin/env python3
"""What the memory system allows a launch of config 2's size (34.6 MB at context 32768), read cold from HBM.

    python -m hqmq_amd.bench_ceiling [--launches 96]

Times kernels that only read (hqmq_amd/csrc_bench/read_probes.hip, libhqmq_bench.so), every launch with its own pair
of HIP events, over 16 buffers / caches in rotation (554 MB: none of it is left in the L2s or the Infinity Cache when its
turn comes again):
  * a contiguous 34.6 MB buffer for blocks in {256, 512, 1024, 2048} x threads in {256, 512} x 16-byte loads in
    flight per thread in {2, 4, 8};
  * the same bytes through global_load_lds (memory to LDS), 256 blocks of 512 threads, every wavefront requesting its
    whole share at once or keeping 1, 2 or 3 pieces of 4 KB ahead;
  * the planes of config 2's packed caches with the grid and the per-lane loads of the register-tile attention
    kernel, for n_splits in {16, 32, 64, 128} and rings of 3, 4 and 6 half-steps;
  * an empty kernel (the floor of the event interval).
Prints one table; medians and means over the launches.
"""
import argparse
import ctypes as C
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

import hqmq  # noqa: E402
from hqmq_amd import _lib as L  # noqa: E402

DEV = "cuda:0"
Hq, Hkv, D_H, S, B_R, T = 32, 8, 128, 96, 4, 32768


def read_planes(cache, n_splits, depth=3, waves=8, events=None, sink=None):
    """Launch the plane-reading probe over one packed cache (16+0 layout at d_h 128)."""
    Kc, Vc = cache.K, cache.V
    nbh = Kc.B * Kc.H
    lib = L.bench_lib()
    need = int(lib.hqmq_bench_read_planes_sink_bytes(C.c_int(nbh), C.c_int(n_splits)))
    if sink is None or sink.numel() < need:
        sink = torch.empty(need, dtype=torch.uint8, device=Kc.device)
    e0, e1 = (C.c_void_p(events[0]), C.c_void_p(events[1])) if events else (C.c_void_p(0), C.c_void_p(0))
    rc = lib.hqmq_bench_read_planes(L.ptr(Kc.main), L.ptr(Vc.main), L.ptr(Kc.scale), L.ptr(Vc.scale), L.i64(Kc.t_cap), C.c_int(T),
                                    C.c_int(nbh), C.c_int(n_splits), C.c_int(depth), C.c_int(waves), L.ptr(sink), L.i64(sink.numel()),
                                    e0, e1, L.stream_ptr(Kc.device))
    if rc:
        raise RuntimeError(f"hqmq_bench_read_planes failed ({rc})")
    return sink


def event_times_us(launch, n):
    """Per-launch GPU durations (us) of launch(i, (ev0, ev1)), each with its own pair of HIP events."""
    hip = C.CDLL("libamdhip64.so")
    evs = []
    for _ in range(n):
        a, b = C.c_void_p(), C.c_void_p()
        assert hip.hipEventCreate(C.byref(a)) == 0 and hip.hipEventCreate(C.byref(b)) == 0
        evs.append((a, b))
    for i in range(8):
        launch(i, None)
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(evs):
        launch(i + 8, (a.value, b.value))
    torch.cuda.synchronize()
    out, ms = [], C.c_float()
    for a, b in evs:
        assert hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        out.append(ms.value * 1e3)
        hip.hipEventDestroy(a)
        hip.hipEventDestroy(b)
    return out


def stats(d):
    d = sorted(d)
    return d[len(d) // 2], sum(d) / len(d), d[0]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--launches", type=int, default=96)
    ap.add_argument("--layers", type=int, default=16)
    args = ap.parse_args()
    import bench
    torch.cuda.set_device(0)
    lib = L.bench_lib()
    q = hqmq.HQMQ(n_layers=64, n_heads=Hkv, secondary_size=S, radius_bits=B_R, device=DEV)
    caches, _ = bench.build_layers(q, T, torch.float16, DEV, args.layers)
    nbytes = caches[0].nbytes(T)
    bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=DEV) for _ in range(args.layers)]
    sink = torch.empty(1 << 22, dtype=torch.uint8, device=DEV)
    st = L.stream_ptr(DEV)
    NL, n = args.layers, args.launches

    def ev(e):
        return (C.c_void_p(e[0]), C.c_void_p(e[1])) if e else (C.c_void_p(0), C.c_void_p(0))

    print(f"cold reads of {nbytes} bytes ({args.layers} buffers in rotation), {n} launches each: median / mean / min us, TB/s at the median")
    d = event_times_us(lambda i, e: lib.hqmq_bench_empty(C.c_int(256), C.c_int(512), *ev(e), st), n)
    print("empty kernel, 256 blocks x 512 threads            : %6.2f %6.2f %6.2f" % stats(d))
    for blocks in (256, 512, 1024, 2048):
        for threads in (256, 512):
            for fl in (2, 4, 8):
                d = event_times_us(lambda i, e: lib.hqmq_bench_read_plain(L.ptr(bufs[i % NL]), L.i64(nbytes), C.c_int(blocks), C.c_int(threads),
                                                                          C.c_int(fl), L.ptr(sink), *ev(e), st), n)
                m = stats(d)
                print(f"plain read  blocks {blocks:5d} threads {threads} in flight {fl}  : {m[0]:6.2f} {m[1]:6.2f} {m[2]:6.2f}   {nbytes / m[0] / 1e6:5.2f} TB/s", flush=True)
    lds_bytes = 256 * 8 * 4 * 4096
    for ahead, name in ((99, "all at once"), (1, "1 piece ahead"), (2, "2 pieces ahead"), (3, "3 pieces ahead")):
        d = event_times_us(lambda i, e: lib.hqmq_bench_read_lds(L.ptr(bufs[i % NL]), C.c_int(256), C.c_int(4), C.c_int(ahead), L.ptr(sink), *ev(e), st), n)
        m = stats(d)
        print(f"to LDS, 256 x 512, 4 x 4 KB per wavefront, {name:14s}: {m[0]:6.2f} {m[1]:6.2f} {m[2]:6.2f}   {lds_bytes / m[0] / 1e6:5.2f} TB/s ({lds_bytes} bytes)", flush=True)
    for ns in (16, 32, 64, 128):
        for depth in (3, 4, 6):
            d = event_times_us(lambda i, e: read_planes(caches[i % NL], ns, depth, 8, e, sink), n)
            m = stats(d)
            print(f"planes of the cache, n_splits {ns:3d}, ring of {depth}      : {m[0]:6.2f} {m[1]:6.2f} {m[2]:6.2f}   {nbytes / m[0] / 1e6:5.2f} TB/s", flush=True)


if __name__ == "__main__":
    main()
