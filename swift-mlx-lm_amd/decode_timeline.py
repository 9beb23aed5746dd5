"""Per-workgroup timeline of the decode launches (benchmark config 1: 4-bit, groups of 64, M = 1).

Runs the measurement build of the library (python swift-mlx-lm_amd/build.py --timeline), whose decode rows kernel
writes four 100 MHz time stamps per workgroup (entry, activations staged, first weight words there, exit) and the
hardware ids of the CU it ran on.  The product library carries none of this.  Prints, per launch of a Llama-3-8B
layer (fused gate+up, down, fused q+k+v, o): how workgroups enter over time, how long each waits for its
activations and its first weights, how many are resident over time, and bytes delivered per phase.

    python swift-mlx-lm_amd/decode_timeline.py [--rows-per-wave R --rows-per-pass B] [--rows M]

The first two options override the launch shape of the rows kernel (measurement build only) for a sweep.  --rows M
(5 .. 16) times the small-batch matrix-core kernel on M activation rows instead; its stamps are entry, activations
staged (behind the barrier), first weight words there, end of the K loop, exit.
"""
import argparse
import ctypes as C
import importlib.util
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def load_package():
    spec = importlib.util.spec_from_file_location("mi355_qlinear_pkg", os.path.join(HERE, "__init__.py"),
                                                  submodule_search_locations=[HERE])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[spec.name] = mod
    spec.loader.exec_module(mod)
    return mod


def bf16_bits(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows-per-wave", type=int, default=0)
    ap.add_argument("--rows-per-pass", type=int, default=0)
    ap.add_argument("--rows", type=int, default=1, help="activation rows of the launch")
    ap.add_argument("--brief", action="store_true", help="one line per launch")
    a = ap.parse_args()
    if a.rows_per_wave:
        os.environ["TL_RPW"] = str(a.rows_per_wave)
    if a.rows_per_pass:
        os.environ["TL_BR"] = str(a.rows_per_pass)
    pkg = load_package()
    pkg.LIB_PATH = os.path.join(HERE, "lib", "libmi355_qlinear_timeline.so")
    if not os.path.exists(pkg.LIB_PATH):
        raise SystemExit("build the measurement library first: python swift-mlx-lm_amd/build.py --timeline")
    L = pkg.library()
    L.mi355q_probe_set_timeline.argtypes = [C.c_void_p]
    L.mi355q_probe_set_timeline.restype = None
    ctx = pkg.Context(0)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    rng = np.random.default_rng(1)

    def weight(n, k):
        words = rng.integers(0, 2**32, size=(n, k // 8), dtype=np.uint32)
        s = bf16_bits(np.full((n, k // 64), 0.004, np.float32))
        z = bf16_bits(np.full((n, k // 64), -0.03, np.float32))
        return ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)

    shapes = {"gate+up": [(14336, 4096), (14336, 4096)], "down": [(4096, 14336)],
              "q+k+v": [(4096, 4096), (1024, 4096), (1024, 4096)], "o": [(4096, 4096)]}
    copies = 6                                     # rotated, so that every launch streams its weights from HBM
    for name, mats in shapes.items():
        ws = [[weight(n, k) for n, k in mats] for _ in range(copies)]
        k = mats[0][1]
        x = ctx.upload(bf16_bits(rng.standard_normal((a.rows, k)).astype(np.float32)))
        ys = [ctx.alloc(a.rows * n * 2) for n, _ in mats]
        stream = ctx.stream_create()

        def launch(i):
            if len(mats) == 1:
                ctx.qgemv(ws[i % copies][0], x, pkg.BF16, ys[0], pkg.BF16, a.rows, 0, 0, 0, stream)
            else:
                ctx.batched_qgemm(ws[i % copies], x, pkg.BF16, ys, pkg.BF16, a.rows, 0, 0, stream)

        L.mi355q_probe_set_timeline(None)
        for i in range(12):
            launch(i)
        ctx.synchronize(stream)
        e0, e1 = ctx.event_create(), ctx.event_create()
        ctx.event_record(e0, stream)
        for i in range(60):
            launch(i)
        ctx.event_record(e1, stream)
        ctx.event_synchronize(e1)
        back_to_back = ctx.event_elapsed_ms(e0, e1) * 1e3 / 60
        nwg = 8192
        tl = ctx.alloc(nwg * 6 * 8)
        ctx.fill(tl, 0)
        ctx.synchronize()
        L.mi355q_probe_set_timeline(C.c_void_p(tl.ptr))
        runs = []
        for r in range(5):
            launch(12 + r)
            ctx.synchronize(stream)
            runs.append(tl.download(np.uint64, (nwg, 6)).copy())
        L.mi355q_probe_set_timeline(None)
        if not all((t[:, 3] > 0).any() for t in runs):
            print(f"== {name}: no time stamps: this launch shape is served by a kernel that writes none")
            continue
        spans = [float((t[t[:, 3] > 0][:, 3].max() - t[t[:, 3] > 0][:, 0].min()) / 100.0) for t in runs]
        t = runs[int(np.argsort(spans)[len(spans) // 2])]
        t = t[t[:, 3] > 0]
        n = len(t)
        t0 = t[:, 0].min()
        entry = (t[:, 0] - t0) / 100.0
        staged = (t[:, 1] - t[:, 0]) / 100.0
        first = (t[:, 2] - t[:, 0]) / 100.0
        life = (t[:, 3] - t[:, 0]) / 100.0
        exit_ = (t[:, 3] - t0) / 100.0
        end = float(exit_.max())
        total_bytes = sum(nn * (kk // 2 + kk // 64 * 4) for nn, kk in mats)
        step = ws[0][0].plan_decode_step(a.rows)
        print(f"== {name}: {step.device_kernel}, {n} workgroups of {step.block[0]} threads, {total_bytes / 1e6:.1f} MB of weights; "
              f"{back_to_back:.2f} us a launch back to back; first entry to last exit {end:.2f} us "
              f"(five runs: {', '.join(f'{s:.2f}' for s in spans)})")
        if not a.brief:
            q = lambda v, p: float(np.percentile(v, p))
            print(f"   workgroups entered: 25% by {q(entry, 25):.2f}, 50% by {q(entry, 50):.2f}, 75% by {q(entry, 75):.2f}, all by {entry.max():.2f} us")
            print(f"   entry -> activations staged: median {q(staged, 50):.2f} (10% {q(staged, 10):.2f}, 90% {q(staged, 90):.2f}) us")
            print(f"   entry -> first weight words: median {q(first, 50):.2f} (10% {q(first, 10):.2f}, 90% {q(first, 90):.2f}) us")
            if a.rows > 1:
                loop = (t[:, 5] - t[:, 0]) / 100.0
                print(f"   entry -> end of the K loop:  median {q(loop, 50):.2f} (10% {q(loop, 10):.2f}, 90% {q(loop, 90):.2f}) us")
            print(f"   entry -> exit:               median {q(life, 50):.2f} (10% {q(life, 10):.2f}, 90% {q(life, 90):.2f}) us")
            print(f"   first workgroup to exit leaves at {exit_.min():.2f} us")
            # bytes delivered over time: a workgroup's share of the weights counts as delivered when it exits
            per_wg = total_bytes / n
            marks = np.linspace(0.0, end, 9)
            line = []
            for lo, hi in zip(marks[:-1], marks[1:]):
                done = int(((exit_ > lo) & (exit_ <= hi)).sum())
                resident = int(((entry <= hi) & (exit_ > hi)).sum())
                line.append(f"{lo:.1f}-{hi:.1f} us: {done * per_wg / (hi - lo) / 1e6:.2f} TB/s, {resident} resident after")
            print("   weights retired per interval: " + "; ".join(line))
        for w_ in ws:
            for w in w_:
                w.destroy()
        x.free()
        tl.free()
        for y in ys:
            y.free()


if __name__ == "__main__":
    main()
