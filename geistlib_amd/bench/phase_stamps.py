"""Where the time goes inside k_cand_scan_final: device timestamps of an instrumented build.

    make -C geistlib_amd phase-stamps [STAMP_MASK=0x...]
    GEIST_HIP_LIB_DIR=geistlib_amd/lib/stamps python3 geistlib_amd/bench/phase_stamps.py [--no-pen] [--rows N]
    GEIST_HIP_LIB_DIR=geistlib_amd/lib/stamps python3 geistlib_amd/bench/phase_stamps.py --walk [ROWS]

Workload: 64 x 128256 fp32, T = 0.7, top-k 40 -> top-p 0.9, penalties over 2048 history ids per
row (the default benchmark workload), 21 copies of the batch rotated so that every launch reads
its logits from HBM. Prints, per stamp taken, minimum / median / maximum over the launch's
workgroups in microseconds from the first workgroup's start, for the last of 40 launches, three
times (--rows N: the same on N rows, e.g. 1 for the decode step of one session). Every stamp costs the wavefront that takes it time: the figures of a sparse mask are
closer to the uninstrumented kernel's than those of a dense one.

--walk: the same for k_whole_row_coop (the whole-row top-p walk spread over the row's chunks) on
ROWS (default 16) flat rows of 128256, top-p 0.9: the stamps of the first row's workgroups."""
import ctypes as C
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))

NAMES = {0: "start", 1: "history table built", 2: "logits loaded", 3: "bound T_w known",
         4: "hand-over stored", 5: "stores acknowledged", 6: "arrival counted",
         7: "final stage: start", 8: "final: B known", 12: "final: places taken",
         13: "final: entries penalised", 9: "final: list complete (barrier)",
         14: "final: counted", 15: "final: ranks reduced", 10: "final: ranked (barrier)",
         11: "end"}
ORDER = [0, 1, 2, 3, 4, 5, 6, 7, 8, 12, 13, 9, 14, 15, 10, 11]


WALK_NAMES = {0: "start", 1: "probabilities formed", 2: "sums of the first step added",
              3: "nucleus edge known", 4: "draw located", 5: "last arrival of the count per chunk",
              6: "token written"}


def walk_main(rows):
    import torch
    from geistlib_amd.binding import HipSampler, SampleParams, load_library
    lib = load_library()
    if not hasattr(lib, "geist_hip_walk_stamps_read"):
        sys.exit("this library takes no stamps: build `make -C geistlib_amd phase-stamps` and set "
                 "GEIST_HIP_LIB_DIR=geistlib_amd/lib/stamps")
    lib.geist_hip_walk_stamps_read.argtypes = [C.c_void_p, C.c_size_t]
    vocab = 128256
    hs = HipSampler(rows, vocab)
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    xs = [torch.randn(rows, vocab, device="cuda", generator=g) * 0.5 for _ in range(4)]
    u = torch.rand(rows, device="cuda", generator=g)
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    prm = SampleParams.make(temperature=1.0, top_p=0.9)
    hs.set_whole_row_walk(1)
    for i in range(10):
        hs.sample(hs.rows(xs[i % 4]), prm, u, out)
    hs.sync()
    buf = (C.c_ulonglong * (64 * 32))()
    if lib.geist_hip_walk_stamps_read(buf, 64 * 32) != 0:
        sys.exit("reading the stamps failed")
    wgs = (vocab + 8191) // 8192
    a = np.frombuffer(buf, dtype=np.uint64).reshape(64, 32).astype(np.int64)[:wgs]
    d = (a - a[:, 0].min()) / 100.0
    print(f"{rows} rows; the first row's {wgs} workgroups; microseconds from their start")
    part = ["histogram sent", "arrived last", "result seen"]
    for k in list(range(7)) + list(range(8, 26)):
        col = d[:, k][(a[:, k] != 0) & (d[:, k] >= 0)]   # (stamps of earlier launches lie before the start)
        if col.size == 0:
            continue
        name = WALK_NAMES.get(k) or f"level {(k - 8) // 3 + 1 if k < 17 else (k - 17) // 3 + 4}: " \
                                    f"{part[(k - 8) % 3 if k < 17 else (k - 17) % 3]}"
        print(f"  {name:<38} min {col.min():6.2f}  median {np.median(col):6.2f}  "
              f"max {col.max():6.2f}  (n = {col.size})")
    print("paths:", sorted(set(hs.row_paths(rows).tolist())), "(4 = walked by the chunks' workgroups)")
    hs.close()


def main():
    if "--walk" in sys.argv:
        rest = [a for a in sys.argv[sys.argv.index("--walk") + 1:] if a.isdigit()]
        return walk_main(int(rest[0]) if rest else 16)
    import torch
    from geistlib_amd.binding import HipSampler, SampleParams, load_library
    lib = load_library()
    if not hasattr(lib, "geist_hip_phase_stamps_read"):
        sys.exit("this library takes no stamps: build `make -C geistlib_amd phase-stamps` and set "
                 "GEIST_HIP_LIB_DIR=geistlib_amd/lib/stamps")
    lib.geist_hip_phase_stamps_read.argtypes = [C.c_void_p, C.c_size_t]
    rows, vocab, hist_n = 64, 128256, 2048
    if "--rows" in sys.argv:
        rows = int(sys.argv[sys.argv.index("--rows") + 1])
    pen = "--no-pen" not in sys.argv
    hs = HipSampler(rows, vocab)
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    copies = [torch.randn(rows, vocab, device="cuda", generator=g) * 2.0 for _ in range(21)]
    u = torch.rand(rows, device="cuda", generator=g)
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    zipf = np.random.default_rng(0).zipf(1.1, (rows, hist_n)) % vocab
    hist = torch.from_numpy(zipf.astype(np.int32)).cuda()
    hlen = torch.full((rows,), hist_n, dtype=torch.int32, device="cuda")
    kw = dict(rep=1.1, freq=0.5, pres=0.3) if pen else {}
    prm = SampleParams.make(temperature=0.7, top_k=40, top_p=0.9, **kw)
    hs.set_logits_hint(True)
    n = 4096 * 16
    buf = (C.c_ulonglong * n)()
    wgs = ((rows + 7) & ~7) * ((vocab + 32767) // 32768)   # the grid holds the rows in eights
    for rep in range(3):
        for i in range(40):
            hs.sample(hs.rows(copies[i % 21], hist if pen else None, hlen if pen else None), prm,
                      u, out)
        hs.sync()
        if lib.geist_hip_phase_stamps_read(buf, n) != 0:
            sys.exit("reading the stamps failed")
        a = np.frombuffer(buf, dtype=np.uint64).reshape(-1, 16).astype(np.int64)[:wgs]
        a = a[a[:, 0] != 0]                      # (the workgroups of the grid's padding take none)
        wgs_run = a.shape[0]
        d = (a - a[:, 0].min()) / 100.0          # the device's clock ticks at 100 MHz
        print(f"run {rep}: {wgs_run} workgroups; microseconds from the first workgroup's start")
        for k in ORDER:
            col = d[:, k]
            col = col[col > 0] if k else col
            if col.size == 0:
                continue
            print(f"  {NAMES[k]:<32} min {col.min():6.2f}  median {np.median(col):6.2f}  "
                  f"max {col.max():6.2f}  (n = {col.size})")
    print("paths of the last launch (0 = served by the hand-over):",
          sorted(set(hs.topk_paths(rows).tolist())))
    hs.close()


if __name__ == "__main__":
    main()
