"""The cost model behind the library's default tile (beam_default_config), its timing table and its fit.

The library picks a tile for a problem without measuring anything: every CU works through
ceil(tiles / CUs) workgroups, `occ` of them at a time (what LDS allows); a workgroup costs a fixed
start-up / epilogue time plus its flops at the per-CU rate of its tile shape, which is higher when
several workgroups share the CU.  Three constants per candidate tile (rate alone, rate with a full CU,
fixed cost) are fitted to `default_tile_timings.json`: microseconds per launch of every candidate on 39
shapes from 512^3 to 8192^3 (square, skinny, short-K), fp16, N(0,1)/sqrt(K) operands, best of two rounds
of 40 launches each, on one MI355X.  `PARAMS` below are the constants compiled into the library
(csrc/capi.hip, kCandidates); a test keeps the two in step.

    python -m beam.default_tile_fit              model's pick per shape against the table, mean / worst regret
    python -m beam.default_tile_fit --refit      coordinate search from PARAMS (what produced them)
    python -m beam.default_tile_fit --collect F  re-measure the table on the GPU at hand into file F
    python -m beam.default_tile_fit --split      the same for calls with a workspace (split-K): pick against sweep
    python -m beam.default_tile_fit --collect-split F   re-measure the split-K sweep into file F
    python -m beam.default_tile_fit --ln         the GEMM+LayerNorm model's pick per shape against its table
    python -m beam.default_tile_fit --fit-ln     least-squares fit of that model's constants to the table
    python -m beam.default_tile_fit --collect-ln F      re-measure that table into file F

With a workspace (beam_gemmrc_splitk, split_k <= 0, no tile given) the deep-pipeline candidates are priced with
their K slices (`auto_slices`) and the reduction; `splitk_timings.json` holds, for 25 shapes from 64x64x8192 to
1024x1024x32768, microseconds per call (one launch) of every tile up to 128x128 x {3+2 slots, deep} x
S in {4, 8, 16, 32, 64} (uniform operands, best of two rounds of 100 calls, one MI355X, the library as shipped:
one launch or two as it decides): the model's pick is what
`predict_split` restates, and a test keeps it in step with the library.

A GEMM+LayerNorm call without a tile (one-kernel form) has a model of its own: one tile per workgroup, each ending
in the epilogue's chain of latencies, so the cost is rounds x (fixed + a tile's flops / rate) with whole rounds.
`ln_tile_timings.json` holds microseconds per call of the one-kernel form with every compiled tile (3 + 2 slots) on 34
shapes (fp16, N(0,1)/sqrt(K), best of two rounds, one MI355X; "default": the library's pick at the time, "plain": the
plain GEMM); `LN_PARAMS` are the least-squares constants compiled into the library (csrc/capi.hip, kLnCandidates).

This stands where the reference has fixed default shapes (cuda/cutlass_kernels/cutlass_gemmrc.cu:22-24).
"""
import json
import math
import os
import random
import sys

CUS = 256
TIMINGS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "default_tile_timings.json")

# name -> (block_m, block_n, workgroups a CU holds at once)
CANDIDATES = {
    "256x256_w128x64": (256, 256, 1), "224x256_w112x64": (224, 256, 1), "192x256_w96x64": (192, 256, 1),
    "256x128_w64x64": (256, 128, 1), "128x256_w64x64": (128, 256, 1), "128x128_w64x64": (128, 128, 2),
    "128x128_w64x32_deep": (128, 128, 1), "128x64_w64x32": (128, 64, 2), "128x64_w64x32_deep": (128, 64, 1),
    "64x64_w32x32": (64, 64, 4), "64x64_w32x32_deep": (64, 64, 1), "64x128_w32x64": (64, 128, 2),
    "64x128_w32x64_deep": (64, 128, 1),
}
# name -> (TFLOP/s per CU alone, with a full CU, fixed microseconds per workgroup slot)
PARAMS = {
    "256x256_w128x64": (6.04, 6.04, 8.0), "224x256_w112x64": (5.95, 5.95, 8.0), "192x256_w96x64": (5.22, 5.22, 8.0),
    "256x128_w64x64": (4.99, 4.99, 6.0), "128x256_w64x64": (4.8, 4.8, 6.0), "128x128_w64x64": (3.8, 4.4, 3.42),
    "128x128_w64x32_deep": (4.05, 4.05, 4.0), "128x64_w64x32": (2.6, 3.4, 3.5), "128x64_w64x32_deep": (3.2, 3.2, 4.2),
    "64x64_w32x32": (1.87, 2.9, 2.7), "64x64_w32x32_deep": (2.4, 2.4, 4.0), "64x128_w32x64": (3.15, 3.4, 3.5),
    "64x128_w32x64_deep": (3.3, 3.3, 4.0),
}


SPLIT_TIMINGS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "splitk_timings.json")
# deep-pipeline candidates (the ones priced with K slices): name -> wavefront tile
SPLIT_WAVES = {"128x128_w64x32_deep": (64, 32), "128x64_w64x32_deep": (64, 32), "64x64_w32x32_deep": (32, 32),
               "64x128_w32x64_deep": (32, 64)}
SPLIT_FIXED_US = 2.0          # the reducing workgroups start behind the multiplying ones
SPLIT_BYTES_PER_US = 2.0e6    # partial sums written through to memory and read back, ~4 TB/s each way


def auto_slices(tiles, K, cus=CUS):
    """Slices the library takes for `tiles` output tiles (csrc/capi.hip: auto_slices)."""
    if tiles * 2 > cus:
        return 1
    ktiles = (K + 63) // 64
    s = min(cus // max(tiles, 1), ktiles // 4, 64)
    half_round = (cus // 2 + tiles - 1) // max(tiles, 1)
    s = min(s, max(ktiles // 16, half_round))
    return max(s, 1)


def predict_split(params, M, N, K):
    """(block_m, block_n, pipeline, slices) of the model's pick for a call with a workspace and no slice count."""
    best = None
    for name, (bm, bn, occ) in CANDIDATES.items():
        alone, full, fixed = params[name]
        tiles = math.ceil(M / bm) * math.ceil(N / bn)
        s = auto_slices(tiles, K) if name in SPLIT_WAVES else 1
        load = math.ceil(tiles * s / CUS)
        conc = min(occ, load)
        rate = alone if occ == 1 else alone + (full - alone) * (conc - 1) / (occ - 1)
        mflop = 2.0e-6 * bm * bn * K / s
        us = math.ceil(load / occ) * fixed + load * mflop / rate
        if s > 1:
            us += SPLIT_FIXED_US + s * M * N * 4.0 / SPLIT_BYTES_PER_US
        if best is None or us < best[0]:
            best = (us, name, bm, bn, s, tiles)
    _, name, bm, bn, s, tiles = best
    pipeline = 2 if name.endswith("_deep") else 0
    if s > 1 and tiles * s <= CUS // 2:
        pipeline = 0   # slices on at most half the CUs: the short queue
    return bm, bn, pipeline, s


def split_regret(params, timings, rows=None):
    """(geometric-mean, worst) ratio of the pick's measured time to the best of the sweep, over the shapes whose
    pick is in the sweep (its slice counts are powers of two)."""
    total, worst, n = 0.0, 0.0, 0
    for key, row in timings.items():
        M, N, K = map(int, key.split("x"))
        bm, bn, pipe, s = predict_split(params, M, N, K)
        t = row.get(f"{bm}x{bn}_p{pipe}_S{s}")
        best_name = min(row, key=row.get)
        if rows is not None:
            rows.append((key, f"{bm}x{bn}_p{pipe}_S{s}", t, best_name, row[best_name]))
        if t is None:
            continue
        r = t / row[best_name]
        total += math.log(r)
        worst = max(worst, r)
        n += 1
    return math.exp(total / max(n, 1)), worst, n


def collect_split(path):
    """Times every tile up to 128x128 x {3+2, deep} x S in {4..64} on the sweep's shapes on the GPU at hand."""
    from . import _C
    out = {}
    tiles = [(64, 64, 32, 32), (64, 128, 32, 64), (128, 64, 64, 32), (128, 128, 64, 32)]
    for key in load_timings(SPLIT_TIMINGS):
        M, N, K = map(int, key.split("x"))
        a = _C.DeviceArray.from_numpy(_C.host_uniform((M, K), _C.F16, 11, 0))
        b = _C.DeviceArray.from_numpy(_C.host_uniform((N, K), _C.F16, 11, 1))
        c = _C.DeviceArray((M, N))
        res = {}
        for (bm, bn, tm, tn) in tiles:
            for pipe in (0, 2):
                pc = _C.TileConfig(bm, bn, tm, tn, pipe, 0)
                for s in (4, 8, 16, 32, 64):
                    if K // 64 // s < 2:
                        continue
                    try:
                        us = min(_C.bench(1, a, b, c, config=pc, split_k=s, warmup=20, iters=100) for _ in range(2)) * 1e3
                    except _C.BeamError:
                        continue
                    res[f"{bm}x{bn}_p{pipe}_S{s}"] = round(us, 2)
        for x in (a, b, c):
            x.free()
        out[key] = res
        print(key, min(res, key=res.get), min(res.values()), flush=True)
    with open(path, "w") as f:
        f.write("{\n" + ",\n".join(f' "{k}": {json.dumps(v)}' for k, v in out.items()) + "\n}\n")


def load_timings(path=TIMINGS):
    with open(path) as f:
        return json.load(f)


def predict(params, M, N, K):
    """(modelled microseconds, candidate name) of the model's pick for a call without a workspace."""
    best = None
    for name, (bm, bn, occ) in CANDIDATES.items():
        alone, full, fixed = params[name]
        tiles = math.ceil(M / bm) * math.ceil(N / bn)
        load = math.ceil(tiles / CUS)
        conc = min(occ, load)
        rate = alone if occ == 1 else alone + (full - alone) * (conc - 1) / (occ - 1)
        mflop = 2.0e-6 * bm * bn * K
        us = math.ceil(load / occ) * fixed + load * mflop / rate
        if best is None or us < best[0]:
            best = (us, name)
    return best


def regret(params, timings, rows=None):
    """(geometric-mean, worst) ratio of the picked candidate's measured time to the best time of any tile."""
    total, worst = 0.0, 0.0
    for key, row in timings.items():
        M, N, K = map(int, key.split("x"))
        us, name = predict(params, M, N, K)
        best = row["best_of_all_tiles"][1]
        r = row["candidates"][name] / best
        total += math.log(r)
        worst = max(worst, r)
        if rows is not None:
            rows.append((key, name, row["candidates"][name], us, row["best_of_all_tiles"][0], best, r))
    return math.exp(total / len(timings)), worst


def refit(params, timings, steps=4000, seed=1):
    """Coordinate search: nudge one constant at a time, keep what lowers the worst, then the mean regret."""
    rng = random.Random(seed)
    params = dict(params)
    best = regret(params, timings)
    for _ in range(steps):
        name = rng.choice(list(params))
        idx = rng.randrange(3)
        old = params[name]
        new = list(old)
        new[idx] *= rng.choice([0.9, 0.95, 1.05, 1.1])
        if CANDIDATES[name][2] == 1 and idx < 2:
            new[0] = new[1] = new[idx]   # one workgroup per CU: one rate
        params[name] = tuple(new)
        r = regret(params, timings)
        if (r[1], r[0]) < (best[1], best[0]) or (r[0] < best[0] and r[1] <= best[1] * 1.001):
            best = r
        else:
            params[name] = old
    return params, best


LN_TIMINGS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ln_tile_timings.json")
# name -> (TFLOP/s per CU, fixed microseconds per round of workgroups); order = the library's candidate order.
# Two candidates share the 256 x 256 tile: the 4-wavefront kernel (one wavefront per SIMD: the faster K loop, and an
# epilogue in which nothing overlaps the vector work of its one wavefront) and the 8-wavefront one (two wavefronts per
# SIMD cover each other's waits in the epilogue): the first wins where K is long, the second where rounds are short.
LN_PARAMS = {
    "256x256_w128x128": (7.91, 18.17), "256x256_w128x64": (7.08, 14.13), "224x256_w112x64": (6.94, 12.35),
    "192x256_w96x64": (6.66, 11.01), "256x128_w64x64": (5.38, 8.00), "128x256_w64x64": (5.41, 8.17),
    "128x128_w64x32": (5.05, 6.65), "64x128_w32x64": (3.33, 3.54), "64x64_w32x32": (2.98, 2.76),
}
LN_FIT_COLUMN = {}
W4_MIN_K = 192


def ln_w4_applies(name, N, K):
    """The 4-wavefront kernel's own conditions (gemm_w4.h); any other candidate: True."""
    return name != "256x256_w128x128" or (K % 64 == 0 and K >= W4_MIN_K and N % 8 == 0)


def _ln_block(name):
    bm, bn = name.split("_w")[0].split("x")
    return int(bm), int(bn)


def ln_fused_applies(name, N, cus=CUS):
    """The one-kernel form's conditions that depend on the tile: 256 CUs, at most 64 column tiles, and the band's
    statistics fit the kernel's LDS ((3 + 2 slots) x 64 K elements x 2 bytes x (block_m, block_n) rows)."""
    bm, bn = _ln_block(name)
    tiles_n = -(-N // bn)
    lds = (3 * bm + 2 * bn) * 128
    return cus == 256 and tiles_n <= 64 and (tiles_n + 1) * bm * 8 <= lds


def ln_rounds(M, N, bm, bn, cus=CUS):
    """Rounds of workgroups of the one-kernel form: a band's column tiles wait for each other, so a band that
    straddles two rounds costs both; a round is worth the whole bands it holds."""
    tiles_m, tiles_n = -(-M // bm), -(-N // bn)
    per_round = max(1, cus // tiles_n)
    return -(-tiles_m // per_round)


def predict_ln(params, M, N, K, cus=CUS):
    """(name, modelled us) of the tile the library takes for the one-kernel GEMM+LayerNorm, None where none applies."""
    best = None
    for name, (rate, fixed) in params.items():
        if not ln_fused_applies(name, N, cus) or not ln_w4_applies(name, N, K):
            continue
        bm, bn = _ln_block(name)
        rounds = ln_rounds(M, N, bm, bn, cus)
        us = rounds * (fixed + 2.0e-6 * bm * bn * K / rate)
        if best is None or us < best[1]:
            best = (name, us)
    return best


def ln_regret(params, table, rows=None):
    logs, worst = [], 1.0
    for key, row in table.items():
        M, N, K = map(int, key.split("x"))
        tiles = {k: v for k, v in row.items() if k not in ("default", "plain")}
        name, us = predict_ln(params, M, N, K)
        t = min(tiles[name], tiles.get(LN_FIT_COLUMN.get(name, name), 1e9))
        bname = min(tiles, key=tiles.get)
        r = t / tiles[bname]
        logs.append(math.log(r))
        worst = max(worst, r)
        if rows is not None:
            rows.append((key, name, t, us, bname, tiles[bname], r, row.get("plain")))
    return math.exp(sum(logs) / len(logs)), worst


def fit_ln(table):
    """Per tile, weighted least squares of measured us on (rounds, rounds x flops of a tile): relative errors."""
    import numpy as np
    out = {}
    for name in LN_PARAMS:
        col = LN_FIT_COLUMN.get(name, name)
        X, y = [], []
        for key, row in table.items():
            if col not in row:
                continue
            M, N, K = map(int, key.split("x"))
            if not ln_w4_applies(name, N, K):
                continue
            bm, bn = _ln_block(name)
            tiles = -(-M // bm) * -(-N // bn)
            if tiles < CUS // 2:  # (a tile is not in question where it leaves most of the device idle)
                continue
            rounds = ln_rounds(M, N, bm, bn, CUS)
            X.append([rounds, rounds * 2.0e-6 * bm * bn * K])
            y.append(row[col])
        X, y = np.array(X), np.array(y)
        coef = np.linalg.lstsq(X / y[:, None], np.ones(len(y)), rcond=None)[0]
        out[name] = (round(float(1.0 / coef[1]), 2), round(float(coef[0]), 2))
    return out


def collect_ln(path):
    """Times the one-kernel GEMM+LayerNorm with every compiled tile on the table's shapes on the GPU at hand."""
    from . import _C
    out = {}
    for key in json.load(open(LN_TIMINGS)):
        M, N, K = map(int, key.split("x"))
        a = _C.DeviceArray.from_numpy(_C.host_normal((M, K), _C.F16, 7, 0, 0.0, K ** -0.5))
        b = _C.DeviceArray.from_numpy(_C.host_normal((N, K), _C.F16, 7, 1, 0.0, K ** -0.5))
        g = _C.DeviceArray.from_numpy(_C.host_normal((N,), _C.F16, 7, 2, 1.0, 0.1))
        bt = _C.DeviceArray.from_numpy(_C.host_normal((N,), _C.F16, 7, 3, 0.0, 0.1))
        c = _C.DeviceArray((M, N))
        n = max(40, int(6000 / max(1.0, 2.0 * M * N * K / 1.2e9)))
        row = {}
        for cfg in _C.list_configs():
            t = _C.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, 0, 0)
            try:
                row[t.name] = round(min(_C.bench(_C.OP_GEMM_LN, a, b, c, gamma=g, beta=bt, config=t, warmup=n, iters=n,
                                                 ln_mode=_C.LN_FUSED) for _ in range(2)) * 1e3, 2)
            except _C.BeamError:
                continue
        row["default"] = round(min(_C.bench(_C.OP_GEMM_LN, a, b, c, gamma=g, beta=bt, warmup=n, iters=n) for _ in range(2)) * 1e3, 2)
        row["plain"] = round(min(_C.bench(_C.OP_GEMM, a, b, c, warmup=n, iters=n) for _ in range(2)) * 1e3, 2)
        for x in (a, b, g, bt, c):
            x.free()
        out[key] = row
        print(key, "plain", row["plain"], "default", row["default"], flush=True)
        with open(path, "w") as f:
            json.dump(out, f, indent=0)


def collect(path):
    """Times every compiled tile (both pipeline depths) on the table's shapes on the GPU at hand."""
    from . import _C
    out = {}
    for key in load_timings():
        M, N, K = map(int, key.split("x"))
        a = _C.DeviceArray.from_numpy(_C.host_normal((M, K), _C.F16, 1, 0, 0.0, K ** -0.5))
        b = _C.DeviceArray.from_numpy(_C.host_normal((N, K), _C.F16, 1, 1, 0.0, K ** -0.5))
        c = _C.DeviceArray((M, N))
        res = {}
        for _ in range(2):
            for cfg in _C.list_configs():
                for pipe in (0, 2):
                    pc = _C.TileConfig(cfg.block_m, cfg.block_n, cfg.wave_m, cfg.wave_n, pipe, 0)
                    try:
                        us = _C.bench(0, a, b, c, config=pc, warmup=20, iters=40) * 1e3
                    except _C.BeamError:
                        continue
                    res[pc.name] = min(res.get(pc.name, 1e9), us)
        for x in (a, b, c):
            x.free()
        name = min(res, key=res.get)
        out[key] = {"candidates": {n: round(res[n], 2) for n in CANDIDATES},
                    "best_of_all_tiles": [name, round(res[name], 2)]}
        print(key, out[key]["best_of_all_tiles"], flush=True)
    with open(path, "w") as f:
        f.write("{\n" + ",\n".join(f' "{k}": {json.dumps(v)}' for k, v in out.items()) + "\n}\n")


def main(argv):
    if argv[:1] == ["--collect"]:
        collect(argv[1])
        return 0
    if argv[:1] == ["--collect-split"]:
        collect_split(argv[1])
        return 0
    if argv[:1] == ["--collect-ln"]:
        collect_ln(argv[1])
        return 0
    if argv[:1] in (["--ln"], ["--fit-ln"]):
        table = json.load(open(LN_TIMINGS))
        params = LN_PARAMS
        if argv[0] == "--fit-ln":
            params = fit_ln(table)
            for name, (rate, fixed) in params.items():
                print(f"{name:22s} {rate:.2f} {fixed:.2f}")
        rows = []
        mean, worst = ln_regret(params, table, rows)
        print("| shape | model's pick | measured us | modelled us | best tile of all | its us | pick / best | plain GEMM us |")
        print("|---|---|---|---|---|---|---|---|")
        for key, name, t, us, bname, bt, r, plain in rows:
            print(f"| {key} | {name} | {t:.1f} | {us:.1f} | {bname} | {bt:.1f} | {r:.3f} | {plain} |")
        print(f"geometric mean {mean:.4f}, worst {worst:.3f} over {len(rows)} shapes")
        return 0
    if argv[:1] == ["--split"]:
        rows = []
        mean, worst, n = split_regret(PARAMS, load_timings(SPLIT_TIMINGS), rows)
        print("| shape | model's pick | its us | best of the sweep | its us |")
        print("|---|---|---|---|---|")
        for key, pick, t, bname, bt in rows:
            print(f"| {key} | {pick} | {'-' if t is None else f'{t:.2f}'} | {bname} | {bt:.2f} |")
        print(f"geometric mean {mean:.4f}, worst {worst:.3f} over {n} shapes whose pick is in the sweep")
        return 0
    timings = load_timings()
    params = PARAMS
    if argv[:1] == ["--refit"]:
        params, _ = refit(PARAMS, timings)
        for name, p in params.items():
            print(f"{name:22s} {p[0]:.2f} {p[1]:.2f} {p[2]:.2f}")
    rows = []
    mean, worst = regret(params, timings, rows)
    print("| shape | model's pick | measured us | modelled us | best tile of all | its us | pick / best |")
    print("|---|---|---|---|---|---|---|")
    for key, name, t, us, bname, bt, r in rows:
        print(f"| {key} | {name} | {t:.1f} | {us:.1f} | {bname} | {bt:.1f} | {r:.3f} |")
    print(f"geometric mean {mean:.4f}, worst {worst:.3f} over {len(rows)} shapes")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
