#!/usr/bin/env python3
"""Benchmark of the alias-method hot path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input that is already resident in HBM:
  c1, c2, c5  offline alias tables for every vertex (sky_alias_build_all), then a biased DeepWalk of length 80
              from the batch of start vertices (sky_walk_offline), and for c5 also PPR (stop 0.15, at most 100 steps)
  c3          online biased 2-hop sampling (sky_sample_online): tables built on the fly for the frontier
  c4          online node2vec (sky_walk_online): first-order tables of every row rebuilt, then rejection sampling
The timed steps run without any per-kernel event; the per-kernel figures of the roofline come from extra, untimed
steps with the library's build profile switched on.  Prints ONE JSON line.  Only one GPU is ever used.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X published

# name -> (scale, edge_factor, weight kind, wa, wb, graph seed, walkers, walk length, ppr)
CONFIGS = {
    "c1": dict(scale=16, ef=16, wkind="uniform", wa=1.0, wb=100.0, seed=42, walkers=4096, length=80, ppr=False),
    "c2": dict(scale=20, ef=16, wkind="unit", wa=0.0, wb=0.0, seed=1, walkers=40000, length=80, ppr=False),
    # online configurations: tables are built on the fly, nothing is built beforehand
    "c3": dict(scale=22, ef=32, wkind="lognormal", wa=0.0, wb=1.0, seed=3, walkers=40000, length=0, ppr=False,
               mode="sage", fanout=[1, 25, 10]),
    "c4": dict(scale=24, ef=16, wkind="uniform", wa=1.0, wb=100.0, seed=4, walkers=40000, length=80, ppr=False,
               mode="node2vec", p=2.0, q=0.5),
    "c5": dict(scale=26, ef=28, wkind="lognormal", wa=0.0, wb=2.0, seed=5, walkers=1000000, length=80, ppr=True),
    # graphs the build was not tuned on (builder-run): another R-MAT shape of the same edge count, and a graph whose
    # rows fill every degree class of the build with the same number of entries
    "rmat25": dict(scale=25, ef=56, wkind="lognormal", wa=0.0, wb=2.0, seed=6, walkers=1000000, length=80, ppr=False),
    "classes": dict(degrees="classes", per_class=50_000_000, wkind="lognormal", wa=0.0, wb=2.0, seed=7, walkers=1000000,
                    length=80, ppr=False),
}
# degree ranges of the build's classes (skywalker_amd/csrc/sky_build.hip, degree_class)
CLASS_RANGES = ([(1, 2), (3, 8), (9, 16), (17, 32), (33, 64), (65, 128), (129, 160), (161, 192), (193, 253), (254, 381), (382, 509), (510, 765), (766, 1021)] +
                [(512 * (nw - 1) - 2, 512 * nw - 3) for nw in range(3, 11)] +
                [(5118, 8189), (8190, 24576), (24577, 65533), (65534, 524287), (524288, 1200000)])


def class_degrees(per_class, seed):
    """Row lengths that put about per_class entries into every degree class, in random order."""
    import numpy as np
    rng = np.random.default_rng(seed)
    parts = []
    for lo, hi in CLASS_RANGES:
        n = max(1, int(per_class / ((lo + hi) / 2)))
        parts.append(rng.integers(lo, hi + 1, n, dtype=np.int64))
    degs = np.concatenate(parts)
    rng.shuffle(degs)
    xadj = np.zeros(len(degs) + 1, np.uint32)
    total = np.cumsum(degs)
    assert total[-1] < 0xFFFFFFFF
    xadj[1:] = total
    return xadj
# algorithmic bytes per edge of one launch: read w (4) and write prob + alias (8); the two tiled passes that only
# read the weights count 4; xadj / valid are per vertex and small
BYTES_PER_EDGE = {"tiled_sum": 4, "tiled_totals": 4}
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "c5_kernel_traffic.txt")
# measured HBM bytes of one whole batch of the online configurations (sum over the batch's kernels)
BATCH_TRAFFIC_FILE = {"c3": os.path.join(ROOT, "profiles", "c3_batch_traffic.txt"),
                      "c4": os.path.join(ROOT, "profiles", "c4_batch_traffic.txt")}
METRIC = "sampled edges/sec (SEPS) + alias-table build edges/sec on 1 MI355X; % HBM peak"
ARITHMETIC = "f64 classification and exact three-limb sums, u64 fixed-point ledger, f32 tables, u32 indices"
KERNEL_OF = {  # build_profile entry -> kernel symbol
    "bin": "bin_count_kernel+bin_scatter_kernel", "small": "small_rows_kernel", "lds_w1": "build_merge_kernel<64,4>",
    "lds_w2": "build_merge_kernel<64,8>", "lds_w6": "build_merge_kernel<64,6>", "mw2_6": "build_merge_kernel<128,6>",
    "tiled_rows": "tiled_rows_kernel+tiled_map_kernel", "tiled_sum": "tiled_sum_kernel+tiled_ledger_kernel",
    "tiled_totals": "tiled_totals_kernel", "tiled_emit": "tiled_scan_kernel+tiled_emit_kernel",
    "streamed": "huge_prefix_kernel+build_huge_kernel", "stream": "build_stream_kernel", "hold": "build_hold_kernel",
}
KERNEL_OF.update({"g%d%s" % (g, x): "build_group_kernel<%d,%d>" % (g, 6 if x else 4)
                  for g in (2, 4, 8, 16, 32) for x in ("", "x")})
KERNEL_OF.update({"g32s": "build_group_kernel<32,5>"})
KERNEL_OF.update({"mw%d" % nw: "build_merge_kernel<%d,8>" % (64 * nw) for nw in range(2, 11)})
KERNEL_OF.update({"mw3": "build_merge_kernel<256,6>", "mw5": "build_merge_kernel<256,10>", "mw6": "build_merge_kernel<512,6>",
                  "mw7": "build_merge_kernel<256,14>", "mw9": "build_merge_kernel<768,6>", "mw10": "build_merge_kernel<512,10>"})


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def oracle_flags():
    """Compiler flags of the CPU oracle, as its Makefile states them."""
    try:
        for line in open(os.path.join(ROOT, "oracle", "Makefile")):
            if line.startswith("CXXFLAGS"):
                return line.split("=", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def load_traffic():
    """profiles/c5_kernel_traffic.txt: measured HBM bytes per edge (per step for the walk) of every kernel, with the
    commit and the commands they come from.  Returns (dict kernel -> bytes, header dict) or (None, None)."""
    try:
        table, head = {}, {}
        for line in open(TRAFFIC_FILE):
            line = line.rstrip("\n")
            if line.startswith("#"):
                if ":" in line:
                    k, v = line[1:].split(":", 1)
                    head[k.strip()] = v.strip()
                continue
            if line.strip():
                k, v = line.split("\t")
                table[k] = float(v)
        return table, head
    except (OSError, ValueError):
        return None, None


def load_batch_traffic(config):
    """profiles/<config>_batch_traffic.txt: `bytes_per_batch <n>` plus header lines `# key: value`.
    Returns (bytes, header dict) or (None, None)."""
    try:
        head, val = {}, None
        for line in open(BATCH_TRAFFIC_FILE[config]):
            line = line.strip()
            if line.startswith("#"):
                if ":" in line:
                    k, v = line[1:].split(":", 1)
                    head[k.strip()] = v.strip()
            elif line.startswith("bytes_per_batch"):
                val = float(line.split()[1])
        return val, head
    except (OSError, ValueError, KeyError, IndexError):
        return None, None


def cpu_baseline_offline(capi, orc, g, cfg, seeds_d, budget_edges=2_000_000_000, walk_sample=1_000_000):
    """Oracle timed on the host cores, on a bounded sample of the same workload."""
    import numpy as np
    V, E = g.V, g.E
    xadj, adjncy, w = g.download()
    # build sample: the leading vertex range holding at most budget_edges edges
    vs = int(np.searchsorted(xadj, min(E, budget_edges), side="right") - 1)
    vs = max(vs, 1)
    es = int(xadj[vs])
    t0 = time.perf_counter()
    orc.alias_build(np.ascontiguousarray(xadj[:vs + 1]), np.ascontiguousarray(w[:es]))
    t_build = time.perf_counter() - t0
    prob, alias, _ = g.tables()
    seeds = seeds_d.to_host()[:walk_sample]
    t0 = time.perf_counter()
    _, _, sampled = orc.walk_offline(xadj, adjncy, prob, alias, seeds, cfg["length"], 0.0, cfg["seed"])
    t_walk = time.perf_counter() - t0
    value = (es + sampled) / (t_build + t_walk)
    return {
        "value": value, "unit": "edges/s", "cores": orc.num_threads(), "cpu": cpu_model(), "kind": "port",
        "compiler_flags": oracle_flags(),
        "sample": "oracle (C++/OpenMP) on the same graph: alias build of vertices [0,%d) = %d edges in %.3f s "
                  "(%.3e edges/s); DeepWalk L=%d of the first %d walkers = %d steps in %.3f s (%.3e steps/s)" %
                  (vs, es, t_build, es / t_build, cfg["length"], len(seeds), sampled, t_walk, sampled / t_walk),
        "build_edges_per_s": es / t_build, "walk_seps": sampled / t_walk,
    }


def online_bench(args, cfg, capi, g, seeds, name, cus, t_gen, torch):
    """Configs 3 and 4: online 2-hop sampling / online node2vec.  A step = one whole batch."""
    import numpy as np
    N = cfg["walkers"]
    if cfg["mode"] == "sage":
        lps, slen = capi.sample_layout(cfg["fanout"])
        out = (capi.DeviceArray(N * lps, np.uint32, fill=capi.FILL), capi.DeviceArray(N * slen, np.uint32, fill=0))
        run = lambda: g.sample_online(seeds, cfg["fanout"], cfg["seed"], out=out)
        what = "online biased %d-hop sampling, fanout %s, with replacement" % (len(cfg["fanout"]) - 1, cfg["fanout"][1:])
    else:
        L = cfg["length"]
        out = (capi.DeviceArray(N * (L + 1), np.uint32, fill=capi.FILL), capi.DeviceArray(N, np.uint32, fill=0))
        if args.n2v_table:
            run = lambda: g.walk_online(capi.BIAS_NODE2VEC, cfg["p"], cfg["q"], seeds, L, 0.0, cfg["seed"], out=out)
            how = "second-order table built per (walker, step)"
        else:
            # every step pays for the first-order tables of the whole graph again, then walks by rejection
            def run():
                bsec = g.build_tables()
                r = g.walk_online(capi.BIAS_NODE2VEC_REJECT, cfg["p"], cfg["q"], seeds, L, 0.0, cfg["seed"], out=out)
                return r[0], r[1], r[2], r[3] + bsec
            how = "first-order tables of all rows rebuilt in every step + rejection on them"
        what = "online node2vec p=%g q=%g, walk length %d (%s)" % (cfg["p"], cfg["q"], L, how)
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    capi.synchronize()
    t0 = time.perf_counter()
    rec = [run() for _ in range(args.steps)]
    torch.cuda.synchronize()
    capi.synchronize()
    wall = (time.perf_counter() - t0) / args.steps
    sampled, ksec = rec[-1][2], sum(r[3] for r in rec) / len(rec)

    # algorithmic bytes of one batch, from the batch's own output
    xadj = g.download_xadj()
    deg = np.diff(xadj.astype(np.int64))
    if cfg["mode"] == "sage":
        data = out[0].to_host((N, lps))
        fan = cfg["fanout"]
        offs, width, o = [], [], 0
        wd = 1
        for f in fan:
            wd *= f
            offs.append(o)
            width.append(wd)
            o += wd
        per_slot, rows = 0, []
        for h in range(len(fan) - 1):
            front = data[:, offs[h]:offs[h] + width[h]].ravel()
            front = front[front < g.V]
            d = deg[front]
            k = fan[h + 1]
            # per frontier vertex of degree d > 0: row bounds 8, weights 4 d, min(k, d) neighbour ids read and written
            per_slot += int((8 + 4 * d[d > 0] + 8 * np.minimum(d[d > 0], k)).sum())
            rows.append(np.unique(front))
        distinct = np.unique(np.concatenate(rows)) if rows else np.zeros(0, np.int64)
        # what one batch must move at least when every distinct frontier row is built once (as this library does):
        # 12 bytes per entry of those rows + 8 per row, + 8 per sampled edge.  The per-slot formula of a sampler that
        # rebuilds a row for every frontier slot that holds it counts the same row many times over: kept as detail.
        distinct_bytes = int(12 * deg[distinct].sum() + 8 * len(distinct)) + 8 * int(sampled)
        alg_bytes = distinct_bytes
        detail = {"formula": "12 per entry and 8 per row of the distinct frontier rows (each built once) + 8 per sampled edge",
                  "distinct_rows_built": int(len(distinct)), "distinct_row_edges": int(deg[distinct].sum()),
                  "per_slot_formula": "sum over frontier slots of 8 + 4 d + 8 min(k, d)",
                  "per_slot_bytes": per_slot, "per_slot_frac": per_slot / ksec / HBM_PEAK}
        kernel = "one batch: frontier_collect_kernel, the build kernels of the frontier rows, sample_hop_kernel (per hop)"
    else:
        steps = sampled
        if args.n2v_table:
            paths = out[0].to_host((N, L + 1))
            lens = out[1].to_host()
            cur = paths[:, :-1]
            prev = np.concatenate([paths[:, :1], paths[:, :-2]], axis=1)
            mask = np.arange(L)[None, :] < lens[:, None]
            dc = deg[np.where(mask, cur, 0)]
            dp = deg[np.where(mask, prev, 0)]
            dp[:, 0] = 0
            alg_bytes = int(((12 + 8 * dc + 4 * dp) * mask).sum())
            detail = {"formula": "sum over steps of 12 + 8 d + 4 d_prev"}
            kernel = "n2v_step_kernel (one launch per step)"
        else:
            alg_bytes = 12 * g.E + 5 * g.V + 24 * steps
            detail = {"formula": "12 E + 5 V (first-order tables) + 24 per step; the rejection trials' reads "
                                 "(12 + 4 log2 d_prev each) are not counted: a lower bound"}
            kernel = "one batch: the offline build kernels, walk_n2v_reject_group_kernel"
    traffic, thead = (None, None) if args.n2v_table else load_batch_traffic(args.config)
    roofline = {"bound": "hbm", "kernel": kernel, "achieved": alg_bytes / ksec / 1e9, "peak": HBM_PEAK / 1e9,
                "unit": "GB/s", "frac": alg_bytes / ksec / HBM_PEAK, "traffic": traffic,
                "traffic_source": ("%s (commit %s)" % (os.path.relpath(BATCH_TRAFFIC_FILE[args.config], ROOT),
                                                       thead.get("commit", "?"))) if traffic else None,
                "launch_ms": ksec * 1e3, "algorithmic_bytes_per_launch": alg_bytes, "detail": detail}

    cpu = None
    if not args.no_cpu:
        from oracle import orc
        hx, hadj, hw = g.download()
        hseeds = seeds.to_host()
        t0 = time.perf_counter()
        if cfg["mode"] == "sage":
            _, _, osampled = orc.sample_online(hx, hadj, hw, hseeds, cfg["fanout"], cfg["seed"])
            what_cpu = "oracle sample_online of the whole batch (%d seeds)" % N
        elif args.n2v_table:
            few = 2000
            _, _, osampled = orc.walk_online(hx, hadj, hw, 1, cfg["p"], cfg["q"], hseeds[:few], cfg["length"], 0.0, cfg["seed"])
            what_cpu = "oracle walk_online (table per step) of the first %d walkers" % few
        else:
            prob, alias, _ = orc.alias_build(hx, hw)
            _, _, osampled = orc.walk_node2vec_reject(hx, hadj, prob, alias, cfg["p"], cfg["q"], hseeds, cfg["length"], 0.0,
                                                      cfg["seed"])
            what_cpu = "oracle alias_build of all rows + walk_node2vec_reject of the whole batch"
        dt = time.perf_counter() - t0
        cpu = {"value": osampled / dt, "unit": "edges/s", "cores": orc.num_threads(), "cpu": cpu_model(), "kind": "port",
               "compiler_flags": oracle_flags(),
               "sample": "%s: %d sampled edges in %.3f s" % (what_cpu, osampled, dt)}
    print(json.dumps({
        "metric": METRIC, "metric_detail": "value = sampled edges per second of one whole batch (tables built on the way)",
        "value": sampled / wall, "unit": "edges/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "arithmetic": ARITHMETIC,
        "data": "synthetic",
        "config": {"workload": "%s: R-MAT scale %d ef %d (%d V, %d E), %s weights; %s, %d start vertices" %
                               (args.config, cfg["scale"], cfg["ef"], g.V, g.E, cfg["wkind"], what, N),
                   "device": name, "compute_units": cus, "graph_generation_s": t_gen},
        "sampled_edges": sampled, "kernel_region_ms": ksec * 1e3, "seps_kernel_region": sampled / ksec,
        "roofline": roofline, "cpu_baseline": cpu}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="c5", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--profile-steps", type=int, default=3,
                    help="untimed steps after the timed ones, run with per-kernel HIP events for the roofline")
    ap.add_argument("--no-walk-variants", action="store_true",
                    help="skip the untimed runs of the walk with the walk index and with walker lists")
    ap.add_argument("--n2v-table", action="store_true",
                    help="config c4: build the second-order table of every (walker, step) instead of rejection sampling")
    ap.add_argument("--calibrate", action="store_true",
                    help="first run one plain 1 GiB copy kernel (copy_u32_kernel): known-size reference for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="tuning knob of the library (sky_set_option), e.g. online_coarse_rows=65536; may be repeated")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the multi-GPU path of the reference is out of scope); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch  # device synchronisation brackets only
    from skywalker_amd import capi
    import numpy as np

    cfg = CONFIGS[args.config]
    for opt in args.option:
        name, value = opt.split("=", 1)
        capi.set_option(name, int(value))
    if args.calibrate:
        words = 1 << 28
        a = capi.DeviceArray(words, np.uint32, fill=1)
        b = capi.DeviceArray(words, np.uint32, fill=2)
        capi.device_copy(b, a, words)
        a.free()
        b.free()
    wk = {"uniform": capi.W_UNIFORM, "unit": capi.W_UNIT, "lognormal": capi.W_LOGNORMAL}[cfg["wkind"]]
    name, cus = capi.device_name()
    t_gen = time.perf_counter()
    if cfg.get("degrees") == "classes":
        g = capi.Graph.from_degrees(class_degrees(cfg["per_class"], cfg["seed"]), cfg["seed"], wk, cfg["wa"], cfg["wb"],
                                    cfg["seed"])
        shape = "rows of every degree class of the build, about %d entries per class, neighbours uniform" % cfg["per_class"]
    else:
        g = capi.Graph.rmat(cfg["scale"], cfg["ef"], cfg["seed"], wk, cfg["wa"], cfg["wb"], cfg["seed"])
        shape = "R-MAT scale %d ef %d" % (cfg["scale"], cfg["ef"])
    t_gen = time.perf_counter() - t_gen
    V, E, N, L = g.V, g.E, cfg["walkers"], cfg["length"]
    seeds = g.gen_seeds(cfg["seed"], N)
    if cfg.get("mode") in ("sage", "node2vec"):
        return online_bench(args, cfg, capi, g, seeds, name, cus, t_gen, torch)
    paths = capi.DeviceArray(N * (L + 1), np.uint32, fill=capi.FILL)
    lengths = capi.DeviceArray(N, np.uint32, fill=0)
    if cfg["ppr"]:
        ppr_paths = capi.DeviceArray(N * 101, np.uint32, fill=capi.FILL)
        ppr_lengths = capi.DeviceArray(N, np.uint32, fill=0)

    def sync():
        torch.cuda.synchronize()
        capi.synchronize()

    def step():
        r = {}
        r["build_s"] = g.build_tables()
        _, _, r["walk_edges"], r["walk_s"] = g.walk_offline(seeds, L, 0.0, cfg["seed"], out=(paths, lengths))
        if cfg["ppr"]:
            _, _, r["ppr_edges"], r["ppr_s"] = g.walk_offline(seeds, 100, 0.15, cfg["seed"] + 1,
                                                              out=(ppr_paths, ppr_lengths))
        return r

    for _ in range(args.warmup):
        step()
    sync()
    rec = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        rec.append(step())
    sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    # per-kernel brackets of the build: extra steps, outside the timed region
    prof = {}
    psteps = max(1, args.profile_steps)
    capi.set_option("build_profile", 1)
    for _ in range(psteps):
        g.build_tables()
        for nm, ms, edges in g.build_profile():
            p = prof.setdefault(nm, [0.0, edges])
            p[0] += ms / psteps
    capi.set_option("build_profile", 0)

    # the same walks with the optional 16-byte walk index, and with live walkers handed from launch to launch:
    # outside the timed region, reported beside the default path
    extras = {}
    if not args.no_walk_variants:
        def walk_ms(reps=3):
            return min(g.walk_offline(seeds, L, 0.0, cfg["seed"], out=(paths, lengths))[3] for _ in range(reps)) * 1e3
        g.build_tables()
        base_ms = walk_ms()
        capi.set_option("walk_compact_every", 16)
        compact_ms = walk_ms()
        capi.set_option("walk_compact_every", 0)
        idx_ms = g.build_walk_index() * 1e3
        indexed_ms = walk_ms()
        steps_n = rec[-1]["walk_edges"]
        extras = {"default_ms": base_ms, "walker_lists_every_16_steps_ms": compact_ms,
                  "walk_index": {"build_ms": idx_ms, "bytes_per_edge": 16, "walk_ms": indexed_ms,
                                 "seps": steps_n / (indexed_ms * 1e-3),
                                 "batches_to_pay_for_the_index": idx_ms / max(base_ms - indexed_ms, 1e-9)}}
        g.build_tables()  # leaves the graph without a current index, as the timed steps saw it

    mean = lambda k: sum(r[k] for r in rec) / len(rec)
    build_s, walk_s, walk_edges = mean("build_s"), mean("walk_s"), rec[-1]["walk_edges"]
    work = E + walk_edges + (rec[-1]["ppr_edges"] if cfg["ppr"] else 0)
    build_bytes = 12 * E + 5 * V
    dom = max((k for k in prof if prof[k][1] > 0), key=lambda k: prof[k][0])  # brackets without edges are host round trips
    dom_ms, dom_edges = prof[dom]
    # the binning pass reads xadj twice (8 bytes per vertex) and builds the rows of one or two entries
    dom_bytes = BYTES_PER_EDGE.get(dom, 12) * dom_edges + (8 * V if dom == "bin" else 0)
    # measured HBM traffic: only when the tracked table was made for the kernels that ran here
    traffic_tab, traffic_head = load_traffic()
    ran = sorted(KERNEL_OF.get(k, k) for k in prof)
    traffic, walk_traffic, traffic_src = None, None, None
    if traffic_tab is not None and args.config == "c5":
        listed = sorted(k for k in traffic_tab if k != "walk_offline_kernel")
        if listed == ran:
            traffic = traffic_tab[KERNEL_OF.get(dom, dom)] * dom_edges
            walk_traffic = traffic_tab.get("walk_offline_kernel")
            traffic_src = "profiles/c5_kernel_traffic.txt (commit %s)" % traffic_head.get("commit", "?")
        else:
            traffic_src = "profiles/c5_kernel_traffic.txt lists other kernels than ran: not used"
    out = {
        "metric": METRIC,
        "metric_detail": "value = (alias-table entries built + walk steps sampled) per second of one whole step "
                         "(build, DeepWalk, PPR); the two rates are also given apart under build and walk",
        "value": work / (ms_per_step * 1e-3), "unit": "edges/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64", "arithmetic": ARITHMETIC, "data": "synthetic",
        "config": {"workload": "%s: %s (%d V, %d E), %s weights; offline alias build of all vertices "
                               "+ biased DeepWalk L=%d from %d start vertices%s" %
                               (args.config, shape, V, E, cfg["wkind"], L, N,
                                " + PPR(0.15, max 100)" if cfg["ppr"] else ""),
                   "device": name, "compute_units": cus, "graph_generation_s": t_gen},
        "build": {"edges_per_s": E / build_s, "ms": build_s * 1e3, "algorithmic_bytes": build_bytes,
                  "hbm_frac": build_bytes / build_s / HBM_PEAK,
                  "kernels_from": "%d untimed steps with per-kernel HIP events after the timed steps" % psteps,
                  "kernels": {KERNEL_OF.get(k, k): {"ms": round(v[0], 4), "edges": v[1],
                                                    "GBps": round(BYTES_PER_EDGE.get(k, 12) * v[1] / (v[0] * 1e-3) / 1e9, 1) if v[0] > 0 else 0}
                              for k, v in prof.items()}},
        "walk": {"seps": walk_edges / walk_s, "ms": walk_s * 1e3, "steps": walk_edges,
                 "algorithmic_bytes": 24 * walk_edges, "hbm_frac": 24 * walk_edges / walk_s / HBM_PEAK,
                 "measured_traffic_bytes_per_step": walk_traffic,
                 "hbm_frac_measured_traffic": (walk_traffic * walk_edges / walk_s / HBM_PEAK) if walk_traffic else None,
                 "variants": extras},
        "roofline": {"bound": "hbm", "kernel": KERNEL_OF.get(dom, dom), "achieved": dom_bytes / (dom_ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": dom_bytes / (dom_ms * 1e-3) / HBM_PEAK,
                     "traffic": traffic, "traffic_source": traffic_src,
                     "launch_ms": dom_ms, "algorithmic_bytes_per_launch": dom_bytes},
    }
    if cfg["ppr"]:
        ppr_s, ppr_edges = mean("ppr_s"), rec[-1]["ppr_edges"]
        out["ppr"] = {"seps": ppr_edges / ppr_s, "ms": ppr_s * 1e3, "steps": ppr_edges}
    if not args.no_cpu:
        from oracle import orc
        out["cpu_baseline"] = cpu_baseline_offline(capi, orc, g, cfg, seeds)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
