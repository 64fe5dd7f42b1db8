#!/usr/bin/env python3
"""Where a launch of the LDS-landing attention kernel spends its time: time stamps taken inside the kernel.

    python -m hqmq_amd.build --stamps && python -m hqmq_amd.bench_stamps

Loads hqmq_amd/libhqmq_amd_stamps.so (attention_fast.hip compiled with -DHQMQ_STAMPS: every wavefront records the
100 MHz real-time counter at fixed points and writes the values out at its end) and runs config 2 at context 32768
(32 q / 8 kv heads, d_h 128, batch 1, s96_r4 fp16, 32 splits): one cache replayed ("warm": the planes sit in the L2s and
the Infinity Cache) and 16 caches in rotation ("cold": read from HBM).  Prints, per stamp, the median, the 90th
percentile and the maximum over the launch's 2048 wavefronts, in us since the launch's first wavefront started (median
over six launches), and how far apart the wavefronts of a block finish.
"""
import ctypes as C
import sys
from pathlib import Path

import numpy as np
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

import hqmq_amd._lib as L  # noqa: E402

L._SO = Path(__file__).resolve().parent / "libhqmq_amd_stamps.so"

import bench  # noqa: E402
import hqmq  # noqa: E402
from hqmq_amd import ops  # noqa: E402

DEV, DT = "cuda:0", torch.float16
Hq, Hkv, D, T, NL, NS, WV = 32, 8, 128, 32768, 16, 32, 8
NAMES = ["first instruction", "tables requested", "first half-step requested", "own table share landed", "barrier passed (tables in LDS)",
         "half-step 1 arrived", "half-step 1 done", "half-step 2 arrived", "half-step 2 done", "half-step 3 arrived", "half-step 3 done",
         "half-step 4 arrived", "half-step 4 done", "block's wavefronts in (merge barrier)", "partials written, end", "arguments read"]


def main():
    if not L._SO.exists():
        raise SystemExit(f"{L._SO} is missing: python -m hqmq_amd.build --stamps")
    q = hqmq.HQMQ(n_layers=64, n_heads=Hkv, secondary_size=96, radius_bits=4, device=DEV)
    caches, queries = bench.build_layers(q, T, DT, DEV, NL)
    out = torch.empty_like(queries[0])
    nblk = Hkv * NS
    st = torch.zeros(nblk * WV * 16, dtype=torch.int64, device=DEV)
    lib = L.lib()

    def launch(j):
        ops.attn_fwd(queries[j], caches[j].K, caches[j].V, T, n_splits=NS, out=out, skip_combine=True)

    for mode in ("warm", "cold"):
        acc, skew = [], []
        for rep in range(6):
            j = (rep + 3) % NL if mode == "cold" else 0
            lib.hqmq_debug_set_stamps(C.c_void_p(0))
            for i in range(NL):                              # cold: walk the other caches first; warm: replay the same one
                if mode == "warm":
                    launch(j)
                elif i != j:
                    launch(i)
            torch.cuda.synchronize()
            st.zero_()
            torch.cuda.synchronize()
            lib.hqmq_debug_set_stamps(C.c_void_p(st.data_ptr()))
            launch(j)
            torch.cuda.synchronize()
            s = st.cpu().numpy().reshape(nblk * WV, 16).astype(np.int64)
            acc.append((s - s[:, 0].min()) / 100.0)
            done = s.reshape(nblk, WV, 16)[:, :, 12]
            skew.append(((done - done.min(axis=1, keepdims=True)) / 100.0).mean(axis=0))
        a = np.stack(acc)
        print(f"--- {mode}: us since the first wavefront of the launch started; median / 90 % / max over the wavefronts (median of 6 launches)")
        for i in (0, 15, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14):
            col = a[:, :, i]
            print(f"{NAMES[i]:40s} {np.median(np.median(col, axis=1)):6.2f} {np.median(np.percentile(col, 90, axis=1)):6.2f} {np.median(col.max(axis=1)):6.2f}")
        print("last half-step done, wavefronts 0..7 of a block, after the block's first (mean over blocks, us):", np.round(np.mean(skew, axis=0), 2))
        sys.stdout.flush()
    lib.hqmq_debug_set_stamps(C.c_void_p(0))


if __name__ == "__main__":
    main()
