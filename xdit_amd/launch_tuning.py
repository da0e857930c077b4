"""Measuring and fitting the time estimate behind the library's choice of launch.

For every attention problem the 16-bit and fp8 kernels can be launched in up to six ways: 128, 256
or 384 query rows per workgroup, as a plain launch or with the last round of query tiles balanced
over the compute units.  The C entry points pick one with a small time estimate (`choose_launch`
in `csrc/api.hip`) whose constants were fitted to measurements.  This module is what took the
measurements and made the fit, for whoever re-tunes the constants (another compute-unit count,
another clock, a changed kernel):

    python -m xdit_amd.launch_tuning sweep grid|cross|long|SEED [--fp8] > FILE    # on the GPU
    python -m xdit_amd.launch_tuning evaluate FILE... [--fp8]                     # CPU: loss of the library's choice
    python -m xdit_amd.launch_tuning fit FILE... [--fp8]                          # CPU: new constants

`sweep` times all six options of every problem of a set (each after 70 ms of the same launch, so
that the chip's power management has settled; the shorter of two such measurements) and prints
one JSON object per problem.  `evaluate` asks the library (host arithmetic only) which option it
would pick for each measured problem and reports how much slower that is than the fastest
measured option.  `fit` solves for the constants: weighted non-negative least squares on the
times, then a short random search on the quantity that matters, the loss of the choice.
"""
import json
import math
import random
import sys
import time

ROWS = (128, 256, 384)
CUS = 256   # compute units the measurements were taken on


# ------------------------------------------------------------------------------------ problems
def problem_set(which, fp8):
    """(B, H, Sq, Sk, D) tuples.  grid: self-attention, B*H 2..48 x S 1024..16896; cross: few to
    many heads, 4096..32760 rows on 77..2304 keys; long: 12000..118800 tokens; a number: 70 random
    problems from that seed."""
    dims = (128,) if fp8 else (128, 64)
    shapes = []
    if which == "grid":
        for D in dims:
            for BH in (2, 3, 5, 6, 8, 12, 16, 24, 40, 48):
                for S in (1024, 1536, 2048, 3072, 4608, 8192, 16896):
                    if BH * S * S * D * 4.0 <= 3e12:
                        shapes.append((1, BH, S, S, D))
    elif which == "cross":
        for D in dims:
            for BH in (3, 16, 40):
                for Sq in (4096, 12000, 32760):
                    for Sk in (77, 226, 512, 1152, 2304):
                        shapes.append((1, BH, Sq, Sk, D))
    elif which == "long":
        for D in dims:
            for BH in (1, 2, 3, 5, 8, 12, 24):
                for S in (12000, 20000, 32768, 50000, 75600, 118800):
                    if 1e12 <= BH * S * S * D * 4.0 <= 2.4e13:
                        shapes.append((1, BH, S, S, D))
    else:
        rnd = random.Random(int(which))
        while len(shapes) < 70:
            D = 128 if fp8 else rnd.choice([128, 128, 64, 72, 96])
            BH = rnd.choice([1, 2, 3, 4, 5, 6, 7, 9, 10, 14, 20, 24, 30, 32, 40])
            S = rnd.choice([1200, 1500, 2500, 3000, 4250, 6000, 9472, 12000, 20000])
            Sk = S if rnd.random() < 0.7 else rnd.choice([77, 226, 512, 1152, 2304, 4608])
            if BH * S * Sk * D * 4.0 <= 3e12:
                shapes.append((1, BH, S, Sk, D))
    return shapes


# ------------------------------------------------------------------------------------ measuring
def _settled_us(fn):
    """Median per-call time (HIP events) after at least 70 ms of the same call."""
    import torch
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    dt = max(time.perf_counter() - t0, 2e-5)
    for _ in range(min(int(0.07 / dt) + 5, 4000)):
        fn()
    n = max(8, min(50, int(0.015 / dt)))
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in ev)
    return t[len(t) // 2] * 1e3


def sweep(which, fp8, out=sys.stdout):
    import torch
    from . import ops
    dev = torch.device("cuda:0")
    saved = dict(ops.TUNING)
    try:
        for (B, H, Sq, Sk, D) in problem_set(which, fp8):
            g = torch.Generator().manual_seed(1)
            q, k, v = (torch.randn(B, H, n, D, generator=g).bfloat16().to(dev) for n in (Sq, Sk, Sk))
            kw = {}
            if fp8:
                (q, qd), (k, kd), (v, vd) = (ops.fp8_quant(t) for t in (q, k, v))
                kw = dict(q_descale=qd, k_descale=kd, v_descale=vd)
            res = torch.empty(B, H, Sq, D, dtype=torch.bfloat16, device=dev)
            rec = {"shape": (B, H, Sq, Sk, D), "opts": []}
            for rows in ROWS:
                for bal in (1, 2):
                    ops.TUNING["rows_per_workgroup"], ops.TUNING["balance"] = rows, bal
                    p = ops.launch_plan(q, k)
                    if bal == 2 and p["ranges"] == 0:
                        continue   # no balanced plan for this shape
                    t = min(_settled_us(lambda: ops.attn_fwd(q, k, v, out=res, **kw)) for _ in range(2))
                    rec["opts"].append({"rows": rows, "bal": bal, "t": round(t, 1), "tiles": p["query_tiles"],
                                        "whole": p["whole_tiles"], "ranges": p["ranges"], "len": p["range_len"],
                                        "streamed": p["streamed"], "slots_per_tile": p["slots_per_tile"]})
            print(json.dumps(rec), file=out, flush=True)
            del q, k, v, res
    finally:
        ops.TUNING.update(saved)


# ------------------------------------------------------------------------------------ the estimate
def _classes(fp8):
    """Index of (rows, workgroups sharing the compute unit) in the constant arrays of choose_launch."""
    if fp8:
        return {(384, 1): 0, (256, 1): 1, (128, 3): 2, (128, 2): 3, (128, 1): 4}
    return {(384, 1): 0, (256, 1): 1, (128, 2): 2, (128, 1): 3}


def features(shape, o, fp8):
    """The terms of the estimate for option `o` of a problem: [rate terms | segment terms | balanced
    launch | partial results | constant], as choose_launch forms them."""
    cls = _classes(fp8)
    nc = len(cls)
    _, _, _, Sk, _ = shape
    nt = (Sk + 63) // 64
    R = o["rows"]
    per_cu = (3 if fp8 else 2) if R == 128 else 1
    slots = CUS * per_cu
    T = o["tiles"]
    f = [0.0] * (2 * nc + 3)
    if o["ranges"] == 0:
        rounds = math.ceil(T / slots) if T <= 4 * slots else T / slots + 0.5
        units, segs, c = rounds * nt, rounds, min(per_cu, math.ceil(T / CUS))
    else:
        full = o["whole"] // slots
        rem = T - o["whole"]
        share = max(4, math.ceil(rem * nt / slots))
        units, segs, c = full * nt + share, full + 1, per_cu
        f[2 * nc] = 1.0
        f[2 * nc + 1] = rem * o["slots_per_tile"] * R / CUS * 1e-3   # thousand partial rows per compute unit
    k = cls[(R, c)]
    f[k] = units * R * c * 1e-3
    f[nc + k] = segs * c
    f[2 * nc + 2] = 1.0
    return f


def _load(files, fp8):
    """{kernel: [(shape, [(features, time, rows, bal), ...]), ...]} with kernel 128 / 64 / 'fp8'."""
    data = {}
    for fn in files:
        for line in open(fn):
            r = json.loads(line)
            key = "fp8" if fp8 else (64 if r["shape"][4] <= 64 else 128)
            data.setdefault(key, []).append((r["shape"], [(features(r["shape"], o, fp8), o["t"], o["rows"], o["bal"]) for o in r["opts"]]))
    return data


def _choice_loss(x, problems, plain_only=False):
    import numpy as np
    losses = []
    for _, opts in problems:
        if plain_only:
            opts = [o for o in opts if o[3] == 1]
        chosen = min(opts, key=lambda o: float(np.dot(o[0], x)))
        losses.append(chosen[1] / min(o[1] for o in opts))
    return float(np.mean(losses)), max(losses)


def fit(files, fp8, search_steps=1500):
    import numpy as np
    from scipy.optimize import nnls
    for key, problems in _load(files, fp8).items():
        nc = len(_classes(fp8))
        A, y, w = [], [], []
        for _, opts in problems:
            best = min(o[1] for o in opts)
            best_plain = min(o[1] for o in opts if o[3] == 1)
            for o in opts:   # options that compete for the choice weigh more
                A.append(o[0])
                y.append(o[1])
                w.append(max((best / o[1]) ** 2, (best_plain / o[1]) ** 2 if o[3] == 1 else 0.0))
        A, y = np.array(A), np.array(y)
        W = np.array(w) / y
        x, _ = nnls(A * W[:, None], y * W)
        objective = lambda v: sum(m + 0.1 * mx for m, mx in (_choice_loss(v, problems), _choice_loss(v, problems, True)))
        best_x, best_l = x, objective(x)
        for seed in range(3):
            rnd = random.Random(seed)
            cx, cl = x.copy(), objective(x)
            for _ in range(search_steps):
                trial = cx * (1 + np.array([rnd.gauss(0, 0.03) for _ in cx]))
                for k in range(nc, 2 * nc + 2):
                    trial[k] = max(0.0, cx[k] + rnd.gauss(0, 0.3))
                l = objective(trial)
                if l < cl:
                    cx, cl = trial, l
            if cl < best_l:
                best_x, best_l = cx, cl
        m, mx = _choice_loss(best_x, problems)
        pm, pmx = _choice_loss(best_x, problems, True)
        print("kernel %s, %d problems: rate {%s}  segment {%s}  balanced launch %.2f  partial results %.2f" % (
            key, len(problems), ", ".join("%.2f" % v for v in best_x[:nc]), ", ".join("%.2f" % v for v in best_x[nc:2 * nc]),
            best_x[2 * nc], best_x[2 * nc + 1]))
        print("    choice %.1f %% from the fastest option on average (worst %.0f %%); among plain launches %.1f %% (worst %.0f %%)" % (
            (m - 1) * 100, (mx - 1) * 100, (pm - 1) * 100, (pmx - 1) * 100))


def evaluate(files, fp8):
    """What the library picks today (launch plan for CUS compute units, host arithmetic) against the
    measured options."""
    import ctypes
    from . import _lib
    stats = {}
    for fn in files:
        for line in open(fn):
            r = json.loads(line)
            B, H, Sq, Sk, D = r["shape"]
            a = _lib.AttnArgs()
            a.struct_size = ctypes.sizeof(_lib.AttnArgs)
            a.dtype = _lib.DTYPE_FP8_E4M3FN if fp8 else _lib.DTYPE_BF16
            a.out_dtype = _lib.DTYPE_BF16
            a.B, a.H, a.Sq, a.Sk, a.D = B, H, Sq, Sk, D
            a.softmax_scale = D ** -0.5
            a.cu_count = CUS
            p = _lib.LaunchPlan()
            p.struct_size = ctypes.sizeof(_lib.LaunchPlan)
            _lib.check(_lib.lib().xdit_attn_launch_plan(ctypes.byref(a), ctypes.byref(p)))
            chosen = (p.rows_per_workgroup, 2 if p.ranges else 1)
            t = {(o["rows"], o["bal"]): o["t"] for o in r["opts"]}
            if chosen not in t:
                continue
            best = min(t.values())
            key = "fp8" if fp8 else ("head_dim <= 64" if D <= 64 else "head_dim 72..128")
            s = stats.setdefault(key, {"loss": [], "plain": [], "worst": (1.0, None)})
            s["loss"].append(t[chosen] / best)
            s["plain"].append(min(v for (rows, bal), v in t.items() if bal == 1) / best)
            if t[chosen] / best > s["worst"][0]:
                s["worst"] = (t[chosen] / best, (r["shape"], chosen, t))
    for key, s in stats.items():
        n = len(s["loss"])
        print("%s: %d problems; the library's choice is %.1f %% slower than the fastest option on average, worst %.0f %% %s; "
              "the fastest PLAIN launch is %.0f %% slower on average, worst %.1fx" % (
                  key, n, (sum(s["loss"]) / n - 1) * 100, (max(s["loss"]) - 1) * 100, s["worst"][1][:2] if s["worst"][1] else "",
                  (sum(s["plain"]) / n - 1) * 100, max(s["plain"])))


def main(argv):
    fp8 = "--fp8" in argv
    args = [a for a in argv if a != "--fp8"]
    if len(args) >= 2 and args[0] == "sweep":
        sweep(args[1], fp8)
    elif len(args) >= 2 and args[0] == "fit":
        fit(args[1:], fp8)
    elif len(args) >= 2 and args[0] == "evaluate":
        evaluate(args[1:], fp8)
    else:
        print(__doc__)
        return 2
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
