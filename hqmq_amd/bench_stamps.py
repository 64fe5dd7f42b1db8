#!/usr/bin/env python3
"""Where a launch of the attention kernels spends its time: time stamps taken inside the kernel.

    python -m hqmq_amd.build --stamps && python -m hqmq_amd.bench_stamps                  # config 2, the LDS-landing kernel
    python -m hqmq_amd.build --stamps && python -m hqmq_amd.bench_stamps --blocks 4       # configs 3, 4 or 5: the outlier
                                                                                          # variant of the register-tile kernel, per block

--blocks: every wavefront of the outlier variants records when its block started, when its own tables were stored, when
the block's barrier was passed, when its first half-step started, when its last one was done and when it left the
kernel, together with the CU it ran on (HW_ID, XCC_ID).  Printed: how long a block's prologue takes, the time per
half-step inside the loop, how far apart the wavefronts of a block and the CUs of the launch finish, and the gap
between two blocks on one CU.

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


def blocks(cfg):
    """Block time line of one launch of the outlier variant on config `cfg` (hqmq_amd/bench_configs.py's caches)."""
    if not L._SO.exists():
        raise SystemExit(f"{L._SO} is missing: python -m hqmq_amd.build --stamps")
    from hqmq_amd import bench_configs
    c = bench_configs.setup(cfg)
    B, Hq, Hkv, d, T, lens, lens_dev, cache = c["B"], c["Hq"], c["Hkv"], c["d"], c["T"], c["lens"], c["lens_dev"], c["cache"]
    Q = torch.randn(B, Hq, 1, d, generator=torch.Generator().manual_seed(7)).to(c["dt"]).to(DEV)
    out = torch.empty_like(Q)
    ns = ops.pick_splits(B, Hq, Hkv, 1, T if lens is None else int(lens.max()), lens is not None)
    order = ops.longest_first(lens_dev) if lens is not None else None
    nblk, wv = ns * B * Hkv, 12 if d == 64 else 8
    st = torch.zeros(nblk * wv * 16, dtype=torch.int64, device=DEV)
    lib = L.lib()

    def go():
        hqmq.fused_attention_packed(Q, cache, kv_lens=lens_dev, T_kv=T, n_splits=ns, out=out, batch_order=order)

    for _ in range(20):
        go()
    torch.cuda.synchronize()
    lib.hqmq_debug_set_stamps(C.c_void_p(st.data_ptr()))
    go()
    torch.cuda.synchronize()
    lib.hqmq_debug_set_stamps(C.c_void_p(0))
    s = st.cpu().numpy().reshape(nblk, wv, 16)
    t0 = s[:, :, 8].min()
    us = lambda i: (s[:, :, i] - t0) / 100.0                    # noqa: E731
    t_in, t_loop, t_end, t_out = us(8), us(9), us(10), us(13)
    steps = s[:, :, 7]
    hw = s[:, 0, 11]
    cu = ((hw >> 32) & 15) * 4096 + (hw & 0xff00) // 256       # XCC, then shader engine / array / CU
    pct = lambda a, q: np.percentile(a, q).round(1)             # noqa: E731
    print(c["name"])
    print(f"{nblk} blocks of {wv} wavefronts on {len(set(cu.tolist()))} CUs, n_splits {ns}; the launch ends {t_out.max():.1f} us after its first "
          f"wavefront started (this build's stamps cost a few per cent)")
    rel = lambda i: np.median((s[:, :, i] - s[:, :, 8]) / 100.0)     # noqa: E731
    print(f"a block's prologue, us since its start (median over wavefronts): tables requested {rel(0):.2f}, first tile requested {rel(2):.2f}, "
          f"its sideband entries {rel(1):.2f}, own tables stored {rel(14):.2f}, barrier passed {rel(15):.2f}, first half-step starts {rel(9):.2f}")
    per = (t_end - t_loop) / np.maximum(steps, 1)
    print(f"half-steps per wavefront and block: {steps.mean():.1f}; us per half-step inside the loop: median {np.median(per):.3f}, "
          f"10 % {pct(per, 10)}, 90 % {pct(per, 90)}")
    skew = t_end.max(axis=1) - t_end.min(axis=1)
    print(f"last half-step done, first to last wavefront of a block: median {np.median(skew):.2f} us, 90 % {pct(skew, 90)}, max {skew.max():.2f}; "
          f"per wavefront index, before the block's last: {np.round((t_end - t_end.max(axis=1, keepdims=True)).mean(axis=0), 1).tolist()}")
    print(f"block merge and write-out after the loop: median {np.median(t_out.max(axis=1) - t_end.max(axis=1)):.2f} us")
    b_start, b_end = t_in.min(axis=1), t_out.max(axis=1)
    by = {}
    for i in range(nblk):
        by.setdefault(int(cu[i]), []).append(i)
    last = np.array([max(b_end[i] for i in v) for v in by.values()])
    nb = np.array([len(v) for v in by.values()])
    print(f"blocks per CU {nb.min()} - {nb.max()}; a CU's last block ends at (us): min {last.min():.1f}, 10 % {pct(last, 10)}, median "
          f"{pct(last, 50)}, 90 % {pct(last, 90)}, max {last.max():.1f}")
    gaps = []
    for v in by.values():
        v = sorted(v, key=lambda i: b_start[i])
        gaps += [b_start[j] - b_end[i] for i, j in zip(v, v[1:])]
    if gaps:
        print(f"from a block's end to the start of the next block on its CU: median {np.median(gaps):.2f} us, max {max(gaps):.2f}")
    xcc = (hw >> 32) & 15
    bper = (t_end - t_loop).max(axis=1) / np.maximum(steps.max(axis=1), 1)
    print("us per half-step by XCD:", [round(float(bper[xcc == x].mean()), 3) for x in sorted(set(xcc.tolist()))])


if __name__ == "__main__":
    if "--blocks" in sys.argv:
        blocks(int(sys.argv[sys.argv.index("--blocks") + 1]))
    else:
        main()
