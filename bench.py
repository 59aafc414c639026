#!/usr/bin/env python3
"""Forward-path benchmark on one MI355X.

A step is one forward pass of one synthetic batch through the C++ host classes
(SparseConvNet) on top of libscn_hip.so: grid build, every rule book, gather /
NiN / max-pool / terminal pool / softmax kernels, and the copy of the class
probabilities back to the host.  `value` is measured with the batch's active
sites and input features already in HBM when the timed region starts;
`value_with_input_upload` / `with_input_upload` is the same pass with sites and
features in pinned host memory, uploaded for every batch (the forward time that
also counts the H2D of the inputs); `value_definition` says which is which.

Warm-up batches, timed batches and a tail of untimed batches are ONE pass
through one batch producer: the clock starts when the last warm-up batch is
finished and stops when the last timed batch is, with the producers busy on
both sides of the region.  The line carries the MEDIAN of `--regions` such
regions (the single figures in `ms_per_step_regions`), the other
configurations in `other_configs`, and HBM traffic only while the kernel
sources hash to what the traffic was measured with.

Prints ONE JSON line: active sites/s (value) and samples/s, the roofline of the
kernel -- or the rule-book construction as a whole -- that takes the most GPU
time, the busiest NiN contraction beside it, a per-kernel table, and the CPU
oracle (its -O3 -march=native build, made here) timed on this host's cores.
"""
import argparse
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
# dense MFMA peaks; bf16x3 issues three bf16 MFMAs per useful one
MFMA_PEAK_TFLOPS = {"fp32": 157.3, "bf16": 2500.0, "bf16x3": 2500.0 / 3}
BALANCE_FLOP_PER_BYTE = {k: v * 1e12 / 8e12 for k, v in MFMA_PEAK_TFLOPS.items()}


# HBM bytes per launch (read + written) measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by a
# copy kernel of known size: kept in a file beside the profiles it was taken from, with the commit it was measured at.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_bench.json")


def measured_traffic():
    """{(workload, kernel family, layer): bytes per launch}, the commit of the measurement and the digest of the
    kernel sources it was made with (or {}, None, None)."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return {}, None, None
    table = {(e["workload"], e["kernel"], e["layer"]): e["read_bytes"] + e["written_bytes"] for e in t["entries"]}
    return table, t.get("measured_at_commit"), t.get("csrc_sha256")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=2, help="1..5, the synthetic configs; 2 is the headline one")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--precision", choices=["fp32", "bf16", "bf16x3"], default="fp32")
    ap.add_argument("--seed", type=int, default=2015)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 disables it)")
    ap.add_argument("--calibration-copy-mb", type=int, default=0,
                    help="first launch a plain row copy (gather with identity rules) of this many MB, so that "
                         "hardware byte counters collected over the run can be scaled by a kernel of known traffic")
    ap.add_argument("--distinct-batches", type=int, default=8,
                    help="also time a pass over this many DIFFERENT synthetic batches taken in turn (other seeds, same "
                         "batch size): their site counts differ, so the bounds of the deferred counts are exercised; "
                         "reported beside the headline figure (0 disables it)")
    ap.add_argument("--from-host", action="store_true",
                    help="also time processDataset() on host-resident Pictures (CPU codify + PCIe upload included)")
    ap.add_argument("--producers", type=int, default=10,
                    help="batch-producer threads building grids and rule books ahead of the forward pass (the "
                         "reference's nBatchProducerThreads, 10 by default there too); they share at most five "
                         "streams")
    ap.add_argument("--producer-streams", type=int, default=-1,
                    help="how many of those streams take part (SparseConvNetCUDA::setProducerStreams; 0: all).  HIP "
                         "spreads streams over 4 hardware queues and kernels of streams that share a queue run in "
                         "order: with two forward lanes, two producer streams leave every stream a queue of its "
                         "own.  Default: 2 for the configs whose forward pass is the longer half (2, 4, 5), all "
                         "for those that wait for their batches (1, 3)")
    ap.add_argument("--regions", type=int, default=5,
                    help="timed regions of --steps batches each; value is their median (min and max beside it)")
    ap.add_argument("--other-configs", default="1,3,4,5,4:bf16,5:bf16",
                    help="configurations (number[:precision]) given a short pass each after the headline one, "
                         "reported under other_configs; empty: none")
    ap.add_argument("--other-steps", type=int, default=20, help="timed batches per region of those passes (at most)")
    ap.add_argument("--other-seconds", type=float, default=150.0,
                    help="no further one of those passes is started after this many seconds")
    ap.add_argument("--train", action="store_true",
                    help="time training batches instead (forward, backward pass, momentum step; Pictures on the host, "
                         "processDataset on a TRAINBATCH dataset): an auxiliary line, not the headline metric")
    ap.add_argument("--fused", type=int, choices=[0, 1], default=1,
                    help="1: setFusedConvolutions, a convolution's gather runs inside the next NiN kernel (same "
                         "results bit for bit); 0: the reference's two steps, gather then NiN")
    return ap.parse_args()


def algorithmic_work(layers, ifaces, batch, precision):
    """{(family, layer): (bytes, flops)} per step, from the sizes of one forward
    pass.  N_in / N_out are active sites of the grids, rows include the
    background rows."""
    work = {}
    n0 = ifaces[0]["gridEntries"]
    work[("grid_build", -1)] = (28 * n0, 0)
    esz = 4
    for i, l in enumerate(layers):
        a, b = ifaces[i], ifaces[i + 1]
        k = l["kind"]
        if k in ("conv", "conv_tri", "maxpool", "maxpool_tri"):
            width = b["nRules"] // max(b["rows"], 1)
            work[("rules", i)] = (12 * a["gridEntries"] + 12 * b["gridEntries"] + 4 * width * b["rows"], 0)
            if k.startswith("conv"):
                count = b["nRules"]
                work[("gather", i)] = (4 * count + 2 * esz * count * a["nFeatures"], 0)
            else:
                C = a["nFeatures"]
                work[("maxpool", i)] = (4 * width * b["rows"] + esz * C * width * b["rows"] + 8 * C * b["rows"], 0)
        elif k == "terminal":
            S = b["nRules"] // max(batch, 1)
            work[("rules", i)] = (12 * a["gridEntries"] + 4 * batch * S, 0)
            work[("terminal", i)] = (esz * a["nFeatures"] * a["gridEntries"] + 4 * batch * S + 4 * batch * a["nFeatures"], 0)
        else:
            M, K, N = b["rows"], l["nIn"], l["nOut"]
            asz = 4  # operands are fp32 in HBM in every mode; bf16 rounding happens on the way into LDS
            work[("nin", i)] = (asz * (M * K + K * N) + 4 * (M * N + N), 2 * M * K * N)
            if i > 0 and layers[i - 1]["kind"].startswith("conv"):
                # gather fused in: the rules and the convolution's input rows are read instead of the wide matrix
                src = ifaces[i - 1]
                work[("conv_nin", i)] = (4 * a["nRules"] + asz * (src["rows"] * src["nFeatures"] + K * N) + 4 * (M * N + N),
                                         2 * M * K * N)
    return work


def csrc_digest():
    """sha256 over the sources of libscn_hip.so (names and contents, sorted): what the byte counters were read for."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "sparseconvnet-archived_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h")) or name == "Makefile":
            h.update(name.encode())
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def timed_regions(run, regions):
    """`regions` timed regions one after the other -> (median, min, max, all) of the seconds each took"""
    secs = [run() for _ in range(max(1, regions))]
    return float(np.median(secs)), float(min(secs)), float(max(secs)), secs


def measure(scn, hostapi, synthetic, args, number, precision, headline):
    """One configuration through the pipeline bench.py times.  headline: everything the one JSON line carries for its
    own workload; otherwise a short pass -- throughput with resident and with uploaded inputs, the dominant entry
    and the NiN roofline."""
    cfg = synthetic.config(number, batch=args.batch if headline else None)
    B = cfg.batch
    producers = max(1, args.producers)
    steps = args.steps if headline else max(1, min(args.steps, args.other_steps))
    warmup = args.warmup if headline else min(args.warmup, 5)
    net = hostapi.Net(cfg.dimension, cfg.nInputFeatures, max(cfg.nClasses, 1), threads=producers)
    streams = args.producer_streams
    if streams < 0 or not headline:
        streams = 2 if number in (2, 4, 5) else 0
    net.setProducerStreams(streams)
    cfg.build(net)
    net.setFusedConvolutions(bool(args.fused))
    if precision != "fp32":
        net.setPrecision(scn.BF16 if precision == "bf16" else scn.BF16X3)
    layers = net.layers()
    weights = synthetic.he_normal_weights(layers, args.seed + 1)
    for i, (W, Bv, pr) in weights.items():
        net.set_weights(i, W, Bv, pr)
    samples = synthetic.make_samples(cfg, args.seed)
    S, K, R, bg, feats, nSites = synthetic.codify(samples, cfg.dimension, cfg.lattice, net.inputSpatialSize,
                                                  cfg.nInputFeatures)
    active = int(len(K))
    ctx = scn.Context(handle=net.context_handle())
    dS, dK, dR, dBg, dF = ctx.array(S, np.int32), ctx.array(K, np.int64), ctx.array(R, np.int32), ctx.array(bg, np.int32), ctx.array(feats, np.float32)
    probs = np.zeros((B, max(cfg.nClasses, 1)), np.float32)

    def step():
        net.forward_resident(B, dS.ptr, dK.ptr, dR.ptr, dBg.ptr, active, nSites, dF.ptr, probs)

    if headline and args.calibration_copy_mb > 0:
        # rows of 64 floats copied through the gather kernel with rules 0..n-1:
        # reads n*256 + n*4 bytes, writes n*256 bytes
        n_rows = args.calibration_copy_mb * (1 << 20) // 256
        src = ctx.empty((n_rows, 64), np.float32)
        dst = ctx.empty((n_rows, 64), np.float32)
        ident = ctx.array(np.arange(n_rows, dtype=np.int32))
        scn.lib().scn_fill32(ctx.h, src.ptr, 0x3F800000, n_rows * 64)
        ctx.gather_rows(src, dst, ident, n_rows, 64)
        ctx.sync()
        print("calibration copy: %d rows of 256 B: read %d B, written %d B" % (n_rows, n_rows * 260, n_rows * 256),
              file=sys.stderr)
        del src, dst, ident

    # pinned host copies of the inputs, for the pass that uploads them with every batch
    def pinned(a):
        h = ctx.host_alloc(a.nbytes)
        np.frombuffer(h.buffer(), a.dtype, a.size)[:] = a.reshape(-1)
        return h

    hS, hK, hR, hBg, hF = (pinned(np.ascontiguousarray(x)) for x in
                           (S.astype(np.int32), K.astype(np.int64), R.astype(np.int32), bg.astype(np.int32),
                            feats.astype(np.float32)))
    # Warm-up, timed and tail batches the way processDataset runs them, in ONE pass: producer threads build grids and
    # rule books on their own streams while the forward lanes run the batches before.  The clock starts when the last
    # warm-up batch is finished and the forward streams are idle, and stops when the last timed batch's probabilities
    # are on the host; `producers` more batches follow untimed, so the producers hold finished batches ready at both
    # ends of the window and have to rebuild during it what the window consumes -- the middle of a long pass.
    # (set-up, before the warm-up: every batch slot's first batch is planned layer by layer and sizes the slot's
    # buffers, its second sizes the staging area of the recorded plans -- three batches per slot leave nothing to
    # allocate)
    priming = 3 * producers
    net.forward_stream_timed(0, priming, B, dS.ptr, dK.ptr, dR.ptr, dBg.ptr, active, nSites, dF.ptr,
                             inputs_on_host=False, h_probs=probs)
    net.setStreamTail(producers)
    ready = []

    def resident_region():
        dt = net.forward_stream_timed(warmup, steps, B, dS.ptr, dK.ptr, dR.ptr, dBg.ptr, active, nSites, dF.ptr,
                                      inputs_on_host=False, h_probs=probs)
        ready.append(net.streamReadyAtStart())
        return dt

    def upload_region():
        return net.forward_stream_timed(warmup, steps, B, hS.ptr, hK.ptr, hR.ptr, hBg.ptr, active, nSites, hF.ptr,
                                        inputs_on_host=True, h_probs=probs)

    regions = args.regions if headline else min(args.regions, 3)
    dt, dt_min, dt_max, dt_all = timed_regions(resident_region, regions)
    ctx.sync()
    ms_per_step = 1e3 * dt / steps
    up, up_min, up_max, up_all = timed_regions(upload_region, regions)
    ctx.sync()
    upload_bytes = int(S.size * 4 + K.size * 8 + R.size * 4 + bg.size * 4 + feats.size * 4)
    with_upload = {"active_sites_per_s": active * steps / up, "samples_per_s": B * steps / up,
                   "ms_per_step": 1e3 * up / steps,
                   "ms_per_step_min_max": [1e3 * up_min / steps, 1e3 * up_max / steps],
                   "bytes_uploaded_per_step": upload_bytes,
                   "note": "sites and features in pinned host memory, uploaded on the producer streams for every "
                           "batch: forward time = rule build + H2D of inputs + all layer kernels + D2H of the "
                           "probabilities (BatchProducer.cu:127-134 inside the clock of SparseConvNetCUDA.cu:277-324)"}
    # the same pass over several different batches taken in turn
    varied = None
    if headline and args.distinct_batches > 1:
        keep, descr, actives = [], [], []
        for i in range(args.distinct_batches):
            Si, Ki, Ri, bgi, fi, ni = synthetic.codify(synthetic.make_samples(cfg, args.seed + 100 + i), cfg.dimension,
                                                       cfg.lattice, net.inputSpatialSize, cfg.nInputFeatures)
            arrs = (ctx.array(Si, np.int32), ctx.array(Ki, np.int64), ctx.array(Ri, np.int32), ctx.array(bgi, np.int32),
                    ctx.array(fi, np.float32))
            keep.append(arrs)
            descr.append((B, arrs[0].ptr, arrs[1].ptr, arrs[2].ptr, arrs[3].ptr, int(len(Ki)), int(ni), arrs[4].ptr))
            actives.append(int(len(Ki)))
        net.setStreamTail(0)
        net.forward_stream_timed_many(0, priming + args.distinct_batches, descr, h_probs=probs)
        net.setStreamTail(producers)
        dv, dv_min, dv_max, _ = timed_regions(
            lambda: net.forward_stream_timed_many(warmup, steps, descr, h_probs=probs), regions)
        ctx.sync()
        timed_sites = sum(actives[(warmup + i) % len(actives)] for i in range(steps))
        varied = {"distinct_batches": args.distinct_batches, "ms_per_step": 1e3 * dv / steps,
                  "ms_per_step_min_max": [1e3 * dv_min / steps, 1e3 * dv_max / steps],
                  "active_sites_per_s": timed_sites / dv, "samples_per_s": B * steps / dv,
                  "active_sites_min_max": [min(actives), max(actives)],
                  "note": "different batches in turn (seeds %d..%d), inputs resident" % (args.seed + 100,
                                                                                        args.seed + 99 + len(actives))}
        del keep
    net.setStreamTail(0)
    # one batch at a time on one stream, nothing overlapped: the latency of a batch
    for _ in range(3):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    ms_latency = 1e3 * (time.perf_counter() - t0) / steps
    mac = hostapi.take_multiply_add_count()  # resets the counter
    step()
    mac = hostapi.take_multiply_add_count()

    # sizes of every interface, for the algorithmic byte / flop counts
    ifaces = []
    for i in range(len(layers) + 1):
        info = net.interface(i, want_features=False)
        ifaces.append(dict(rows=info["nSpatialSites"], nFeatures=info["nFeatures"], nRules=int(info["rules"].size),
                           gridEntries=int(info["grids"][0].size)))
    work = algorithmic_work(layers, ifaces, B, precision)

    # per-kernel durations: HIP events on the library's stream, same steps again
    ctx.prof_reset()
    ctx.prof_enable(True)
    # what a span costs by itself: two events around nothing, and around a kernel of one idle wavefront
    for _ in range(5):
        ctx.prof_probe(False)
    ctx.prof_spans()
    for _ in range(50):
        ctx.prof_probe(False)
    bare = [ms for _, _, ms in ctx.prof_spans()]
    for _ in range(50):
        ctx.prof_probe(True)
    idle = [ms for _, _, ms in ctx.prof_spans()]
    span_floor_ms = float(np.median(bare))
    span_idle_kernel_ms = float(np.median(idle))
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    dt_prof = time.perf_counter() - t0
    spans = ctx.prof_spans()
    ctx.prof_enable(False)
    tot, cnt = {}, {}
    for fam, tag, ms in spans:
        key = (fam, tag)
        tot[key] = tot.get(key, 0.0) + ms
        cnt[key] = cnt.get(key, 0) + 1
    kernels = []
    for key, ms_total in tot.items():
        fam, tag = key
        ms = ms_total / steps
        byts, flops = work.get(key, (0, 0))
        entry = dict(kernel=fam, layer=tag, ms_per_step=round(ms, 5), launches_per_step=cnt[key] / steps)
        if fam in ("gather", "nin", "conv_nin", "maxpool", "terminal", "softmax"):
            # one kernel per span: take off what the two events cost around nothing
            ms = max(ms - span_floor_ms * entry["launches_per_step"], 1e-6)
            entry["ms_kernel"] = round(ms, 5)
        if fam in ("nin", "conv_nin") and flops:
            K_, N_ = layers[tag]["nIn"], layers[tag]["nOut"]
            intensity = flops / max(byts, 1)
            entry["shape"] = [ifaces[tag + 1]["rows"], K_, N_]
            if intensity >= BALANCE_FLOP_PER_BYTE[precision]:
                a = flops / (ms * 1e-3) / 1e12
                entry.update(bound="mfma", achieved=a, peak=MFMA_PEAK_TFLOPS[precision], unit="TFLOP/s")
            else:
                a = byts / (ms * 1e-3) / 1e9
                entry.update(bound="hbm", achieved=a, peak=HBM_PEAK_GBS, unit="GB/s")
        elif byts:
            a = byts / (ms * 1e-3) / 1e9
            entry.update(bound="hbm", achieved=a, peak=HBM_PEAK_GBS, unit="GB/s")
        if "achieved" in entry:
            entry["frac"] = entry["achieved"] / entry["peak"]
            entry["achieved"] = round(entry["achieved"], 3)
            entry["frac"] = round(entry["frac"], 5)
            if entry["bound"] == "hbm" and entry["frac"] > 0.9 and byts < 128e6:
                # a layer of tens of MB that the previous kernel has just written is read from the
                # 256 MB last-level cache: the algorithmic bytes did not all cross the HBM interface
                entry["note"] = "operands resident in the last-level cache; not an HBM-rate measurement"
        kernels.append(entry)
    kernels.sort(key=lambda e: -e["ms_per_step"])
    fam_ms = {}
    for e in kernels:
        fam_ms[e["kernel"]] = fam_ms.get(e["kernel"], 0.0) + e["ms_per_step"]
    # Rule-book construction as a whole (every layer's plan and fill, recorded and run together as two kernels, or
    # layer by layer): a span of it covers several launches, so it is priced as one family against the algorithmic
    # bytes of all rule books of a step
    rule_spans = [e for e in kernels if e["kernel"] == "rules"]
    rules_entry = None
    if rule_spans:
        r_ms = sum(e["ms_per_step"] for e in rule_spans)
        r_launches = sum(e["launches_per_step"] for e in rule_spans)
        r_ms_k = max(r_ms - span_floor_ms * r_launches, 1e-6)
        r_bytes = sum(b_ for (fam, _), (b_, _f) in work.items() if fam == "rules")
        a = r_bytes / (r_ms_k * 1e-3) / 1e9
        rules_entry = dict(kernel="rules", layer="all", ms_per_step=round(r_ms, 5), ms_kernel=round(r_ms_k, 5),
                           launches_per_step=r_launches, bound="hbm", achieved=round(a, 3), peak=HBM_PEAK_GBS,
                           unit="GB/s", frac=round(a / HBM_PEAK_GBS, 5), algorithmic_bytes=int(r_bytes), traffic=None)
        if r_launches <= 2.5:
            rules_entry["note"] = ("every layer's rule book in two launches, one workgroup per sample: all layers' "
                                   "occupancy masks by dilation, then owners, rows and rule rows per output site "
                                   "in LDS; integer work bound by instruction issue on one compute unit per sample, "
                                   "the HBM roofline is far from binding")
        else:
            rules_entry["note"] = ("layer by layer through masks, rank prefixes and rows by rank in HBM: a dozen "
                                   "launches per layer; the rule rows themselves leave at 4-6 TB/s")
    traffic_table, traffic_commit, traffic_digest = measured_traffic()
    default_input = args.seed == 2015 and precision == "fp32" and args.fused == 1 and (not headline or args.batch is None)
    traffic_note = None
    if traffic_table and traffic_digest != csrc_digest():
        # the byte counters were read for other kernels than the ones that ran just now
        traffic_table = {}
        traffic_note = ("the kernel sources have changed since the byte counters in profiles/hbm_traffic_bench.json "
                        "were read (commit %s): no traffic figure is printed" % traffic_commit)
    fused_layers = {e["layer"] for e in kernels if e["kernel"] == "conv_nin"}
    for e in kernels:
        e["traffic"] = traffic_table.get((cfg.name, e["kernel"], e["layer"])) if default_input else None
    if rules_entry and default_input:
        rules_entry["traffic"] = traffic_table.get((cfg.name, "rules", "all"))

    def as_roofline(e):
        r = dict(kernel="%s[layer %s]" % (e["kernel"], e["layer"]), bound=e["bound"], achieved=e["achieved"],
                 peak=e["peak"], unit=e["unit"], frac=e["frac"], traffic=e["traffic"],
                 us_per_step=round(1e3 * e.get("ms_kernel", e["ms_per_step"]), 2))
        if "shape" in e:
            r["shape_MKN"] = e["shape"]
        if "note" in e:
            r["note"] = e["note"]
        return r

    # the dominant entry: whatever takes the most GPU time per step, a single kernel or the rule books as a whole
    single = [e for e in kernels if "achieved" in e and e["kernel"] in ("gather", "nin", "conv_nin", "maxpool", "terminal")]
    candidates = single + ([rules_entry] if rules_entry else [])
    dominant = max(candidates, key=lambda e: e.get("ms_kernel", e["ms_per_step"])) if candidates else None
    roofline = as_roofline(dominant) if dominant else None
    nin_only = [e for e in single if e["kernel"] in ("nin", "conv_nin") and e.get("bound") == "mfma"]
    roofline_nin = as_roofline(max(nin_only, key=lambda e: e["ms_kernel"])) if nin_only else None
    nin_flops = sum(work[(e["kernel"], e["layer"])][1] for e in nin_only)
    nin_ms = sum(e["ms_kernel"] for e in nin_only)
    if roofline_nin and nin_ms > 0:
        roofline_nin["all_mfma_bound_layers"] = dict(
            layers=sorted(e["layer"] for e in nin_only), tflops=round(nin_flops / (nin_ms * 1e-3) / 1e12, 2),
            frac=round(nin_flops / (nin_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS[precision], 4),
            per_layer_frac={str(e["layer"]): e["frac"] for e in sorted(nin_only, key=lambda e: e["layer"])})
    pools = [e for e in single if e["kernel"] == "maxpool"]
    roofline_pool = as_roofline(max(pools, key=lambda e: e["ms_kernel"])) if pools else None

    if not headline:
        net.close()
        return {"workload": cfg.name, "batch": B, "precision": precision, "active_sites": active,
                "steps": steps, "warmup": warmup, "regions": regions,
                "ms_per_step": ms_per_step, "ms_per_step_min_max": [1e3 * dt_min / steps, 1e3 * dt_max / steps],
                "active_sites_per_s": active * steps / dt, "samples_per_s": B * steps / dt,
                "with_input_upload": {k: with_upload[k] for k in ("ms_per_step", "ms_per_step_min_max",
                                                                  "active_sites_per_s", "samples_per_s")},
                "batches_ready_at_t0": ready, "producer_streams_in_use": net_streams(streams, producers),
                "ms_single_batch_latency": ms_latency, "roofline": roofline, "roofline_nin": roofline_nin,
                "roofline_maxpool": roofline_pool,
                "rules": None if not rules_entry else {k: rules_entry[k] for k in
                                                       ("ms_kernel", "launches_per_step", "achieved", "frac",
                                                        "algorithmic_bytes", "traffic")}}

    from_host = None
    if args.from_host:
        # the reference's own entry point: Pictures in host memory, codifyInputData on the producer threads, input
        # sites and features uploaded over PCIe for every batch
        reps = max(2, min(3 * steps, 60))  # enough batches for the pass to outweigh its fill and drain
        ds = hostapi.Dataset(cfg.name, cfg.nInputFeatures, max(cfg.nClasses, 1), hostapi.TESTBATCH)
        for _ in range(reps):
            for pts, f, label in samples:
                ds.add_points(cfg.dimension, cfg.lattice, pts, f, label)
        if net.layers()[-1]["act"] == synthetic.SOFTMAX:
            inUse = net.producerStreamsInUse()
            net.setProducerStreams(0)  # production is the longer half here: every stream
            net.processDataset(ds, B)  # warm-up pass (buffers grow)
            t0 = time.perf_counter()
            net.processDataset(ds, B)
            dth = time.perf_counter() - t0
            net.setProducerStreams(inUse)
            from_host = {"ms_per_batch": 1e3 * dth / reps, "active_sites_per_s": active * reps / dth,
                         "samples_per_s": B * reps / dth, "batches": reps,
                         "producer_streams_in_use": min(5, producers),
                         "note": "processDataset on host Pictures: CPU codify + H2D of sites and features included"}
        ds.close()

    cpu_baseline = None
    if args.cpu_seconds > 0:
        cpu_baseline = cpu_leg(cfg, layers, weights, samples, net.inputSpatialSize, args.cpu_seconds)

    out = {
        "metric": "active sites/sec + samples/sec fwd at 1 GPU; % HBM GB/s and % MFMA peak",
        "value": active * steps / dt,
        "unit": "active sites/s",
        "value_definition": "median of %d timed regions of %d batches each; every region is the middle of one longer "
                            "pass (warm-up before, %d more batches behind it); a batch's sites and features are "
                            "resident in HBM when its region starts; the clock covers grid build, every rule book, "
                            "all layer kernels and the copy of the probabilities to the host" % (regions, steps, producers),
        "value_min_max": [active * steps / dt_max, active * steps / dt_min],
        "samples_per_s": B * steps / dt,
        "value_with_input_upload": with_upload["active_sites_per_s"],
        "with_input_upload": with_upload,
        "varied_batches": varied,
        "producer_streams_in_use": net.producerStreamsInUse(),
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "timed_regions": regions,
        "tail_batches_per_region": producers,
        "batches_ready_at_t0": ready,
        "ms_per_step": ms_per_step,
        "ms_per_step_min_max": [1e3 * dt_min / steps, 1e3 * dt_max / steps],
        "ms_per_step_regions": [round(1e3 * x / steps, 5) for x in dt_all],
        "ms_single_batch_latency": ms_latency,
        "ms_per_step_with_event_timing": 1e3 * dt_prof / steps,
        "event_span_floor_us": round(1e3 * span_floor_ms, 3),
        "event_span_idle_kernel_us": round(1e3 * span_idle_kernel_ms, 3),
        "producer_threads": producers,
        "priming_batches": priming,
        "fused_convolutions": sorted(fused_layers),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if precision == "fp32" else precision,
        "data": "synthetic",
        "config": {"workload": cfg.name, "batch": B, "input_field": net.inputSpatialSize, "lattice": cfg.lattice,
                   "dimension": cfg.dimension, "active_sites": active, "input_rows": nSites,
                   "stack": [list(c) for c in cfg.stack], "precision": precision, "seed": args.seed,
                   "fused": bool(args.fused)},
        "mega_multiply_adds_per_sample": mac / B / 1e6,
        "giga_multiply_adds_per_s": mac / (ms_per_step * 1e-3) / 1e9,
        "roofline": roofline,
        "roofline_nin": roofline_nin,
        "roofline_maxpool": roofline_pool,
        "rules": rules_entry,
        "traffic_measured_at_commit": traffic_commit,
        "traffic_note": traffic_note,
        "kernel_family_ms_per_step": {k: round(v, 5) for k, v in fam_ms.items()},
        "kernels": kernels,
        "cpu_baseline": cpu_baseline,
    }
    if from_host:
        out["from_host_pictures"] = from_host
    net.close()
    return out


def net_streams(wanted, producers):
    pool = min(5, producers)
    return pool if wanted < 1 or wanted > pool else wanted


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (the forward path shards by sample "
              "with no exchange between the GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    # the host classes announce every layer on stdout like the reference does;
    # keep stdout for the one JSON line and send that chatter to stderr
    sys.stdout.flush()
    saved_stdout = os.dup(1)
    os.dup2(2, 1)
    from __graft_entry__ import load_package
    scn = load_package()
    from sparseconvnet_archived_amd import hostapi, synthetic

    if args.train:
        cfg = synthetic.config(args.config, batch=args.batch)
        net = hostapi.Net(cfg.dimension, cfg.nInputFeatures, max(cfg.nClasses, 1), threads=max(1, args.producers))
        net.setProducerStreams(max(0, args.producer_streams))
        cfg.build(net)
        net.setFusedConvolutions(bool(args.fused))
        for i, (W, Bv, pr) in synthetic.he_normal_weights(net.layers(), args.seed + 1).items():
            net.set_weights(i, W, Bv, pr)
        train_leg(args, cfg, net, hostapi, synthetic.make_samples(cfg, args.seed), saved_stdout)
        return
    out = measure(scn, hostapi, synthetic, args, args.config, args.precision, True)
    # the other configurations, a short pass each (the headline config's line stays the line)
    others = []
    t_start = time.perf_counter()
    for item in [x for x in args.other_configs.split(",") if x]:
        number, _, prec = item.partition(":")
        number, prec = int(number), prec or "fp32"
        if number == args.config and prec == args.precision:
            continue
        if time.perf_counter() - t_start > args.other_seconds:
            others.append({"workload": "config %d %s" % (number, prec), "skipped": "time budget of the run"})
            continue
        print("bench.py: config %d, %s" % (number, prec), file=sys.stderr, flush=True)
        others.append(measure(scn, hostapi, synthetic, args, number, prec, False))
    out["other_configs"] = others
    sys.stdout.flush()
    os.dup2(saved_stdout, 1)
    print(json.dumps(out))


def train_leg(args, cfg, net, hostapi, samples, saved_stdout):
    """--train: `warmup` untimed training batches, then `steps` timed ones, through processDataset on a TRAINBATCH
    dataset of the same synthetic samples (learning rate 1e-4, momentum 0.9)."""
    assert cfg.nClasses > 1, "training needs a net that ends in the classifier (configs 2, 3, 4)"
    B = cfg.batch

    def dataset(nBatches):
        ds = hostapi.Dataset("train", cfg.nInputFeatures, cfg.nClasses, hostapi.TRAINBATCH)
        for _ in range(nBatches):
            for pts, f, label in samples:
                ds.add_points(cfg.dimension, cfg.lattice, pts, f, label)
        return ds

    net.processDatasetTrain(dataset(max(1, args.warmup)), B, 1e-4, 0.9)
    timed = dataset(args.steps)
    t0 = time.perf_counter()
    nll = net.processDatasetTrain(timed, B, 1e-4, 0.9)
    dt = time.perf_counter() - t0
    line = {
        "metric": "training samples/s (forward + backward + momentum step, 1 GPU)", "value": B * args.steps / dt,
        "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * dt / args.steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s, batch %d, training batches from host-resident Pictures" % (cfg.name, B),
                   "mode": "train", "learning_rate": 1e-4, "momentum": 0.9, "nll_of_the_timed_pass": nll},
        "roofline": None, "cpu_baseline": None,
    }
    sys.stdout.flush()
    os.dup2(saved_stdout, 1)
    print(json.dumps(line))


def cpu_leg(cfg, layers, weights, samples, spatialSize, budget_s):
    """The CPU oracle on this host's cores, same batch, bounded wall time.  Timed in its -O3 -march=native build,
    made here, on the host whose cores are timed (a library built with -march=native elsewhere may not run here);
    the parity build (-mavx2 -ffp-contract=off) is timed instead if that build fails."""
    odir = os.path.join(ROOT, "oracle")
    flags_var = "CFLAGS"
    try:
        subprocess.check_call(["make", "-C", odir, "-s", "-B", "native"], stdout=subprocess.DEVNULL,
                              stderr=subprocess.DEVNULL)
        os.environ["SCN_ORACLE_LIB"] = os.path.join(odir, "libscn_oracle_native.so")
        flags_var = "CFLAGS_NATIVE"
    except (OSError, subprocess.CalledProcessError):
        pass
    import oracle as orc
    import oracle_net
    from sparseconvnet_archived_amd import synthetic
    # threads used: the host's cores, at most 16 (a one-GPU box's share of its machine)
    nproc = os.cpu_count() or 1
    cores = min(nproc, 16)
    ora = oracle_net.Net(cfg.dimension, cfg.nInputFeatures, max(cfg.nClasses, 1))
    cfg.build(ora)
    for i, (W, Bv, pr) in weights.items():
        ora.set_weights(i, W, Bv, pr)
    # bounded sample: shrink the batch until one pass fits the budget
    sub = samples
    if cfg.number == 5:
        sub = samples[:2]
    elif cfg.number == 4:
        sub = samples[:16]
    S, K, R, bg, feats, n = synthetic.codify(sub, cfg.dimension, cfg.lattice, spatialSize, cfg.nInputFeatures)
    orc.set_threads(cores)
    times, t_start = [], time.perf_counter()
    while len(times) < 2 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        ora.forward(len(sub), S, K, R, bg, feats, n, keep=False)
        times.append(time.perf_counter() - t0)
    full = float(np.median(times))
    # rule books only, one thread (the reference's own CPU code on this path)
    g = orc.Grids.from_flat(len(sub), S, K, R, bg)
    t0 = time.perf_counter()
    cur = g
    for l in ora.layers:
        if l["kind"] in ("conv", "maxpool"):
            cur, _, _ = orc.rules_square(cur, cfg.dimension, l["inSize"], l["outSize"], l["size"], l["stride"], l.get("minActive", 1))
        elif l["kind"] == "terminal":
            cur, _, _ = orc.rules_terminal(cur)
    rules_only = time.perf_counter() - t0
    orc.set_threads(1)
    # the same with T producer-style threads, one batch slot each (BatchProducer.cu:90-106 runs up to 10)
    import threading
    T = min(10, cores)

    def one_slot():
        cur = orc.Grids.from_flat(len(sub), S, K, R, bg)
        for l in ora.layers:
            if l["kind"] in ("conv", "maxpool"):
                cur, _, _ = orc.rules_square(cur, cfg.dimension, l["inSize"], l["outSize"], l["size"], l["stride"],
                                             l.get("minActive", 1))
            elif l["kind"] == "terminal":
                cur, _, _ = orc.rules_terminal(cur)

    threads = [threading.Thread(target=one_slot) for _ in range(T)]
    t0 = time.perf_counter()
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    rules_T = time.perf_counter() - t0
    flags = ""
    try:
        for line in open(os.path.join(ROOT, "oracle", "Makefile")):
            if line.split("=", 1)[0].strip() == flags_var:
                flags = line.split("=", 1)[1].strip()
    except OSError:
        pass
    return {"value": len(K) / full, "unit": "active sites/s", "cores": cores, "host_nproc": nproc, "kind": "port",
            "oracle_cflags": flags,
            "sample": "%s, %d of %d samples, %d passes, median" % (cfg.name, len(sub), len(samples), len(times)),
            "ms_per_batch": 1e3 * full, "samples_per_s": len(sub) / full,
            "rulebooks_only_1_thread_ms": 1e3 * rules_only,
            "rulebooks_only_active_sites_per_s": len(K) / rules_only,
            "rulebooks_only_threads": T, "rulebooks_only_T_threads_active_sites_per_s": T * len(K) / rules_T}


if __name__ == "__main__":
    main()
