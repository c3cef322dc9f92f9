#!/usr/bin/env python3
"""Benchmark of the gridding hot path on one MI355X.

A step is one pass over one synthetic batch of 50 ragged complexes
(configurations 1 and 2 of the benchmark definition): per-example rigid transform of the atoms,
forward splat into a 50x28x48^3 float32 tensor, atom-gradient backward against a
N(0,1) upstream gradient and the un-rotation of those gradients.  All inputs are
resident in HBM before the timed region.  One JSON line is printed.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]
                    [--no-write-stream] [--no-graph] [--serial-only] [--no-autotune]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def event_ms(fn, iters, warmup=2):
    """Average milliseconds of fn() over iters launches after `warmup` untimed ones, timed with
    events on the stream the kernels are launched on (torch's current stream)."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def step_breakdown(fns, iters):
    """Average milliseconds of each launch of a step when the launches follow each other as in the
    timed loop (events between them on the launch stream).  A check on the per-kernel figures: a
    kernel that leaves dirty lines in the last-level cache looks shorter here than launched alone
    and the kernel after it longer."""
    import torch
    rows = [[torch.cuda.Event(enable_timing=True) for _ in range(len(fns) + 1)]
            for _ in range(iters)]
    torch.cuda.synchronize()
    for row in rows:
        row[0].record()
        for fn, ev in zip(fns, row[1:]):
            fn()
            ev.record()
    torch.cuda.synchronize()
    return [sum(row[i].elapsed_time(row[i + 1]) for row in rows) / iters
            for i in range(len(fns))]


TRAFFIC_PROFILE = os.path.join("profiles", "bench_kernel_trace_and_traffic.txt")


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 counter summary of this same
    command (FETCH_SIZE + WRITE_SIZE, KiB per dispatch; calibration factor 1.0, stated in that
    file) -- counters cannot be read from inside the run, so this figure is only as fresh as that
    file.  None when the summary is missing or does not list the kernel."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return None
    start = [i for i, l in enumerate(lines) if "FETCH_SIZE_KiB" in l and "WRITE_SIZE_KiB" in l]
    if not start:
        return None
    for l in lines[start[0] + 1:]:
        parts = l.split()
        if len(parts) >= 3 and l.startswith(kernel):
            try:
                return int((float(parts[-2]) + float(parts[-1])) * 1024)
            except ValueError:
                return None
    return None


def forward_traffic():
    """Both launches of a forward call."""
    parts = [measured_traffic("sort_atoms_kernel"), measured_traffic("splat_sorted_kernel")]
    return None if None in parts else sum(parts)


def cpu_baseline(cfg, ntypes, nsample, threads):
    """Oracle (CPU restatement of the reference loops) on the first nsample examples."""
    import oracle
    off = cfg["offsets"][: nsample + 1]
    n = int(off[-1])
    gm = oracle.GridMaker(0.5, 23.5)
    rng = np.random.default_rng(1)
    diff = rng.standard_normal((nsample, ntypes, gm.dim, gm.dim, gm.dim), dtype=np.float32)
    t0 = time.perf_counter()
    moved = oracle.transform_forward_batch(off, cfg["quats"], cfg["centers"], cfg["translations"],
                                           cfg["coords"][:n], nthreads=threads)
    gm.forward_batch(off, cfg["centers"], moved, cfg["types"][:n], cfg["radii"][:n], ntypes,
                     nthreads=threads)
    t1 = time.perf_counter()
    grads = gm.backward_batch(off, cfg["centers"], moved, cfg["types"][:n], cfg["radii"][:n],
                              diff, nthreads=threads)
    oracle.transform_backward_batch(off, cfg["quats"], cfg["centers"], cfg["translations"], grads,
                                    dotranslate=False, nthreads=threads)
    t2 = time.perf_counter()
    return dict(total_s=t2 - t0, forward_s=t1 - t0, backward_s=t2 - t1, atoms=n)


def parity_sample(cfg, gm_args, ntypes, nsample, moved, grid, diff, grads):
    """Distance of the step's results from the CPU oracle on the first `nsample` examples: max
    abs error, max relative error and the number of values outside 1e-6 + 1e-5*|ref|; the atom
    gradients against the oracle's sums in double and against its float loop (the reference's
    order), whose own distance from the sums in double is given beside them."""
    import oracle
    from util import parity_stats
    off = cfg["offsets"][: nsample + 1]
    n = int(off[-1])
    og = oracle.GridMaker(*gm_args)
    m = moved[:n].cpu().numpy()
    ref_moved = oracle.transform_forward_batch(off, cfg["quats"], cfg["centers"],
                                               cfg["translations"], cfg["coords"][:n], nthreads=8)
    ref_grid = og.forward_batch(off, cfg["centers"], ref_moved, cfg["types"][:n], cfg["radii"][:n],
                                ntypes, nthreads=8)
    d = diff[:nsample].cpu().numpy()
    g32 = og.backward_batch(off, cfg["centers"], ref_moved, cfg["types"][:n], cfg["radii"][:n], d,
                            nthreads=8)
    g64 = np.concatenate([og.backward(cfg["centers"][b], ref_moved[off[b]:off[b + 1]],
                                      cfg["types"][off[b]:off[b + 1]],
                                      cfg["radii"][off[b]:off[b + 1]], d[b], f64=True)
                          for b in range(nsample)])
    got_g = grads[:n].cpu().numpy()
    return {
        "sample": "first %d examples (%d atoms) against the CPU oracle" % (nsample, n),
        "tolerance": "1e-6 + 1e-5*|ref|",
        "transform_bit_exact": bool(np.array_equal(m, ref_moved)),
        "forward": parity_stats(grid[:nsample].cpu().numpy(), ref_grid),
        "backward_vs_f64_sums": parity_stats(got_g, g64),
        "backward_vs_float_loop": parity_stats(got_g, g32),
        "float_loop_vs_f64_sums": parity_stats(g32, g64),
    }


def other_workloads(mg, synth, gm, offsets, centers, moved, types, radii, grid, diff, grads,
                    n_atoms, bwd_bytes, small=False):
    """The remaining configurations, one kernel each, events on the launch stream: the backward
    pass with 90 % of the upstream gradient zeroed (configuration 2), vector types into 28x96^3
    for Gaussian and binary density (configuration 3), trilinear resampling under random rotations
    (configuration 4).  Fractions are algorithmic bytes / time against the HBM peak."""
    import torch
    res = {}

    def entry(ms, nbytes, **more):
        gbs = nbytes / (ms * 1e-3) / 1e9
        e = {"ms": round(ms, 4), "GBps": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)}
        e.update(more)
        return e

    # configuration 2, sparse variant: same dense storage, 10 % of the values non-zero
    gen = torch.Generator(device="cuda").manual_seed(2)
    diff.mul_((torch.rand(diff.shape, device="cuda", generator=gen) < 0.1).to(diff.dtype))
    ms = event_ms(lambda: gm.backward_batch(offsets, centers, moved, types, radii, diff, grads), 20)
    res["backward_sparse10"] = entry(ms, bwd_bytes,
                                     atom_grads_per_s=round(n_atoms / (ms * 1e-3), 1))

    # configuration 4: the gridded configuration-1 atoms with N(0, 0.1) noise on 5 % of the
    # voxels, resampled under per-example rotations and +-1.5 A shifts
    B, K, D = grid.shape[0], grid.shape[1], grid.shape[2]
    gm.forward_batch(offsets, centers, moved, types, radii, grid)
    src = diff                                   # reuse the buffer of the upstream gradient
    gen = torch.Generator(device="cuda").manual_seed(4)
    src.normal_(0.0, 0.1, generator=gen)
    src.mul_((torch.rand(src.shape, device="cuda", generator=gen) < 0.05).to(src.dtype))
    src.add_(grid)
    rng = np.random.default_rng(4)
    quats = torch.as_tensor(synth.random_quaternions(rng, B)).cuda()
    shifts = torch.as_tensor(rng.uniform(-1.5, 1.5, (B, 3)).astype(np.float32)).cuda()
    zeros = torch.zeros((B, 3), device="cuda")
    dst = grid                                   # the forward pass's output buffer
    gi = mg.GridInterpolater(0.5, 23.5, 0.5, 23.5)
    ms = event_ms(lambda: gi.forward_batch(src, quats, zeros, shifts, dst), 10)
    res["interpolate"] = entry(ms, 2 * src.numel() * 4, grids_per_s=round(B / (ms * 1e-3), 1),
                               workload="configs[4]: %d x %dx%d^3 gridded atoms + 5 %% noise, "
                                        "random rotation, +-1.5 A" % (B, K, D))

    # configuration 3: 16 x 10,000 atoms with 28-float type vectors into 28x96^3
    VB, VN = (2, 300) if small else (16, 10000)    # small: a dry run of this function, not a figure
    v = synth.vector_batch(nbatch=VB, natoms=VN)
    ab = mg.AtomBatch(v["offsets"])
    ab.dev
    vc, vt, vr = [torch.as_tensor(v[k]).cuda() for k in ("coords", "types", "radii")]
    vcen = torch.as_tensor(v["centers"]).cuda()
    for binary in (False, True):
        gv = mg.GridMaker(0.25, 23.75, binary)
        out = torch.empty((VB,) + gv.grid_dimensions(28), device="cuda")
        ms = event_ms(lambda: gv.forward_batch(ab, vcen, vc, vt, vr, out), 5)
        nbytes = out.numel() * 4 + vc.shape[0] * (16 + 4 * 28)
        key = "forward_vector_binary" if binary else "forward_vector"
        res[key] = entry(ms, nbytes, grids_per_s=round(VB / (ms * 1e-3), 1),
                         workload="configs[3]: %d x %d atoms, 28x96^3 at 0.25 A" % (VB, VN))
        try:
            # the same call without the per-slab atom lists (every workgroup scans every atom of its
            # example): the plain entry point of the C ABI, which takes no workspace
            from libmolgrid_amd import _capi
            off32 = ab.dev
            call = lambda: _capi.check(_capi.lib.mg_forward_vector(
                gv._p, VB, off32.data_ptr(), ab.largest, vcen.data_ptr(), _capi.f3((0, 0, 0)),
                vc.data_ptr(), vt.data_ptr(), vr.data_ptr(), 28, out.data_ptr(),
                torch.cuda.current_stream().cuda_stream), "mg_forward_vector")
            res[key]["without_atom_lists_ms"] = round(event_ms(call, 5), 4)
        except Exception as e:      # a new measurement must not cost the bench line
            res[key]["without_atom_lists_ms"] = repr(e)[:200]
        del out
    try:
        # backward pass for vector types on the same atoms (atom and type gradients): the upstream
        # gradient 16 x 28 x 96^3 is read once
        gv = mg.GridMaker(0.25, 23.75)
        vdiff = torch.randn((VB,) + gv.grid_dimensions(28), device="cuda",
                            generator=torch.Generator(device="cuda").manual_seed(3))
        vag, vtg = torch.empty_like(vc), torch.empty_like(vt)
        ms = event_ms(lambda: gv.backward_batch(ab, vcen, vc, vt, vr, vdiff, vag, vtg), 3, warmup=1)
        res["backward_vector"] = entry(
            ms, vdiff.numel() * 4 + vc.shape[0] * (16 + 4 * 28) + vc.shape[0] * (12 + 4 * 28),
            atom_grads_per_s=round(vc.shape[0] / (ms * 1e-3), 1),
            workload="configs[3] atoms: atom + type gradients against a N(0,1) gradient %dx28x96^3" % VB)
        del vdiff, vag, vtg
    except Exception as e:          # a new measurement must not cost the bench line
        res["backward_vector"] = {"error": repr(e)[:200]}
    try:
        # the autograd layer of the reference's training loop (python/torch_bindings.py:102-136) on the
        # configuration-1 atoms as a padded batch with one-hot type vectors: forward + backward
        from libmolgrid_amd.torch_bindings import Coords2Grid
        off = offsets.host
        width = int(np.diff(off).max())
        pc = torch.zeros((B, width, 3), device="cuda")
        pt = torch.zeros((B, width, K), device="cuda")
        pr = torch.zeros((B, width), device="cuda")
        ti = types.long().clamp(min=0)
        for b in range(B):
            n = int(off[b + 1] - off[b])
            sl = slice(int(off[b]), int(off[b + 1]))
            pc[b, :n], pr[b, :n] = moved[sl], radii[sl]
            pt[b, torch.arange(n, device="cuda"), ti[sl]] = 1.0
        layer = Coords2Grid(gm)
        pc.requires_grad_(True)
        upstream = src                                # any (B,K,D,D,D) tensor of values

        def c2g():
            g_out = layer(pc, pt, pr)
            g_out.backward(upstream)
            pc.grad = None

        ms = event_ms(c2g, 5, warmup=2)
        res["coords2grid_fwd_bwd"] = entry(
            ms, 2 * upstream.numel() * 4 + n_atoms * (16 + 4 * K) * 2,
            grids_per_s=round(B / (ms * 1e-3), 1),
            workload="Coords2Grid layer, padded batch %d x %d atoms, one-hot %d-type vectors, 28x48^3: "
                     "forward + backward (atom and type gradients)" % (B, width, K))
        del pc, pt, pr
    except Exception as e:          # a new measurement must not cost the bench line
        res["coords2grid_fwd_bwd"] = {"error": repr(e)[:200]}
    # the same atoms with radii by type instead of by atom (a density per atom AND channel: no
    # matrix product, 28 times the density evaluations)
    gv = mg.GridMaker(0.25, 23.75, False, True)
    tr = torch.as_tensor(np.random.default_rng(11).uniform(1.2, 2.0, (VB, 28)).astype(np.float32)).cuda()
    out = torch.empty((VB,) + gv.grid_dimensions(28), device="cuda")
    ms = event_ms(lambda: gv.forward_batch(ab, vcen, vc, vt, tr, out), 3, warmup=1)
    res["forward_vector_type_radii"] = entry(
        ms, out.numel() * 4 + vc.shape[0] * (12 + 4 * 28), grids_per_s=round(VB / (ms * 1e-3), 1),
        workload="configs[3] atoms with type-indexed radii (%d x 28 radii), Gaussian" % VB)
    del out
    return res


class Workload(object):
    """The batch of the headline configuration resident in HBM, and the launches of a step."""

    def __init__(self, args):
        import torch
        import libmolgrid_amd as mg
        import synth
        self.torch, self.mg, self.synth, self.args = torch, mg, synth, args
        B, T = args.batch, 28
        self.B, self.T = B, T
        self.cfg = cfg = synth.config1(nbatch=B)
        self.gm = gm = mg.GridMaker(0.5, 23.5)
        self.D = D = gm.get_first_dim()
        self.n_atoms = int(cfg["offsets"][-1])
        # everything resident in HBM before timing
        self.offsets = mg.AtomBatch(cfg["offsets"])
        self.offsets.dev
        self.coords = torch.as_tensor(cfg["coords"]).cuda()
        self.types = torch.as_tensor(cfg["types"]).cuda()
        self.radii = torch.as_tensor(cfg["radii"]).cuda()
        self.quats = torch.as_tensor(cfg["quats"]).cuda()
        self.centers = torch.as_tensor(cfg["centers"]).cuda()
        self.trans = torch.as_tensor(cfg["translations"]).cuda()
        self.moved = torch.empty_like(self.coords)
        self.grid = torch.empty((B, T, D, D, D), device="cuda")
        gen = torch.Generator(device="cuda").manual_seed(1)
        self.diff = torch.randn((B, T, D, D, D), device="cuda", generator=gen)
        self.grads = torch.empty_like(self.coords)
        self.side = None
        # True: the backward launch also takes the gradients back through the example's rotation
        # (mg_backward_index_unrotated: one launch instead of two, the same floats bit for bit)
        self.fused_unrotation = False

    def k_transform(self):
        self.mg.transform_batch(self.offsets, self.quats, self.centers, self.trans, self.coords,
                                self.moved)

    def k_forward(self):
        self.gm.forward_batch(self.offsets, self.centers, self.moved, self.types, self.radii,
                              self.grid)

    def k_forward_no_atoms(self, types_none):
        self.gm.forward_batch(self.offsets, self.centers, self.moved, types_none, self.radii,
                              self.grid)

    def k_backward(self):
        self.gm.backward_batch(self.offsets, self.centers, self.moved, self.types, self.radii,
                               self.diff, self.grads)

    def k_unrotate(self):
        self.mg.transform_batch(self.offsets, self.quats, self.centers, self.trans, self.grads,
                                self.grads, dotranslate=False, inverse=True)

    def k_backward_unrotated(self):
        self.gm.backward_batch(self.offsets, self.centers, self.moved, self.types, self.radii,
                               self.diff, self.grads, unrotate=(self.quats, self.centers))

    def step_serial(self):
        # the reference's order, one stream (k_backward_unrotated does the last two in one
        # launch, bit for bit; it measures the same, see kernels.backward.unrotated_ms)
        self.k_transform()
        self.k_forward()
        self.backward_and_unrotation()

    def backward_and_unrotation(self):
        if self.fused_unrotation:
            self.k_backward_unrotated()
        else:
            self.k_backward()
            self.k_unrotate()

    def step_overlapped(self):
        # The forward and the backward pass of a step do not depend on each other, and the
        # forward pass is two launches: the small sort launch (a chain of dependent phases that
        # fills 40 % of the CUs for 12 us) runs on a second stream beside the backward pass
        # instead of in front of the splat launch.  Same launches, same results.
        torch = self.torch
        if self.side is None:
            self.side = torch.cuda.Stream()       # default priority, like the main stream
            self.ev_moved, self.ev_sorted = torch.cuda.Event(), torch.cuda.Event()
        main = torch.cuda.current_stream()
        self.k_transform()
        self.ev_moved.record(main)
        self.side.wait_event(self.ev_moved)
        with torch.cuda.stream(self.side):
            sb = self.gm.sort_batch(self.offsets, self.centers, self.moved, self.types, self.radii,
                                    self.T)
            self.ev_sorted.record(self.side)
        if self.fused_unrotation:
            self.k_backward_unrotated()
        else:
            self.k_backward()
        main.wait_event(self.ev_sorted)
        self.gm.splat_batch(sb, self.grid)
        if not self.fused_unrotation:
            self.k_unrotate()

    def timed(self, run):
        """(ms per step, ms per step the host needs to enqueue) over exactly --steps steps after
        --warmup untimed ones, device synchronised on both sides."""
        torch, args = self.torch, self.args
        for _ in range(args.warmup):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run()
        t_enqueued = time.perf_counter()          # the host has handed over every launch
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return (t1 - t0) / args.steps * 1e3, (t_enqueued - t0) / args.steps * 1e3


def run_candidates(args):
    """Child process of the benchmark (--candidates): the step in the ways of enqueueing it and
    the write-outs of the splat launch that are not the library's defaults.  One JSON line per
    result, written as soon as it is known, so that whatever a later candidate does -- an error,
    a capture the runtime refuses, the end of the process -- the earlier lines stand and the
    parent's own figures, measured before this process started, are not touched.

    A step can be enqueued in the reference's order on one stream or with the sort beside the
    backward pass, launch by launch or as one captured HIP graph (nothing in a step allocates or
    synchronises), with either write-out.  Every candidate is first checked bit for bit against
    the serial eager step with the default write-out, then timed like it."""
    import torch
    from libmolgrid_amd import _capi
    torch.cuda.set_device(0)
    w = Workload(args)
    grid, grads = w.grid, w.grads

    def emit(d):
        print(json.dumps(d))
        sys.stdout.flush()

    _capi.lib.mg_forward_index_paged(0)
    w.step_serial()
    torch.cuda.synchronize()
    expect = (grid.clone(), grads.clone())

    def same_as_serial(what):
        torch.cuda.synchronize()
        if not (torch.equal(grid, expect[0]) and torch.equal(grads, expect[1])):
            raise RuntimeError("%s differs from the serial eager step" % what)
        grid.zero_()
        grads.zero_()

    def graph_of(fn, what):
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        for _ in range(2):                        # replays must reproduce the eager results
            grid.zero_()
            grads.zero_()
            graph.replay()
            same_as_serial("replay of the captured %s step" % what)
        return graph

    def candidate(name, fn, as_graph):
        try:
            grid.zero_()
            grads.zero_()
            fn()
            same_as_serial(name)
            run = graph_of(fn, name).replay if as_graph else fn
            ms, enq = w.timed(run)
            emit({"candidate": name, "ms_per_step": round(ms, 4), "enqueue_ms_per_step": round(enq, 4)})
        except Exception as e:                    # reported under its name; the others stand
            emit({"candidate": name, "error": repr(e)[:200]})

    it = max(args.steps, 10)
    lib = _capi.lib

    def select(instance):
        lib.mg_forward_index_paged(1 if "paged" in instance else 0)
        lib.mg_forward_index_core_skip(1 if "core" in instance else 0)

    def step_variants(prefix, with_eager):
        if with_eager:
            candidate(prefix + "serial_eager", w.step_serial, False)
        if not args.no_graph:
            candidate(prefix + "serial_graph", w.step_serial, True)
        if not args.serial_only:
            candidate(prefix + "overlapped_eager", w.step_overlapped, False)
            if not args.no_graph:
                candidate(prefix + "overlapped_graph", w.step_overlapped, True)

    # 1. the library's default instance of the splat launch, enqueued the other ways
    select("per_wave")
    step_variants("", False)
    # 2. the other instances of the splat launch -- the paged write-out, tail-only blocks without
    # the exponential, both --: their grids bit for bit, the forward call's time with each, and
    # the store skeleton of either write-out (the same call with every atom ignored)
    valid, check, fastest = [], {}, None
    if not args.no_autotune:
        check = {"identical": {}}
        try:
            w.k_transform()
            check["per_wave_ms"] = round(event_ms(w.k_forward, it), 4)
            torch.cuda.synchronize()
            default_grid = grid.clone()
            types_none = torch.full_like(w.types, -1.0)
            check["per_wave_stores_ms"] = round(event_ms(lambda: w.k_forward_no_atoms(types_none), it), 4)
            for instance in ("core", "paged", "paged_core"):
                try:
                    select(instance)
                    grid.zero_()
                    check[instance + "_ms"] = round(event_ms(w.k_forward, it), 4)
                    torch.cuda.synchronize()
                    check["identical"][instance] = bool(torch.equal(grid, default_grid))
                    if instance == "paged":
                        check["paged_stores_ms"] = round(event_ms(lambda: w.k_forward_no_atoms(types_none), it), 4)
                except Exception as e:
                    check[instance + "_error"] = repr(e)[:200]
                    check["identical"][instance] = False
            del default_grid, types_none
        except Exception as e:
            check["error"] = repr(e)[:200]
        select("per_wave")
        emit({"write_out_check": check})
        # 3. the fastest of them that gives the same grids, enqueued every way
        valid = [i for i in ("core", "paged", "paged_core")
                 if check["identical"].get(i) and (i + "_ms") in check]
        if valid and "per_wave_ms" in check:
            fastest = min(valid, key=lambda i: check[i + "_ms"])
            if check[fastest + "_ms"] < check["per_wave_ms"]:
                select(fastest)
                step_variants(fastest + "/", True)
                select("per_wave")
    # 4. the un-rotation of the gradients inside the backward launch (four launches a step instead
    # of five), with the default instance and with the fastest one
    w.fused_unrotation = True
    step_variants("fused_unrotation/", True)
    if not args.no_autotune and valid and "per_wave_ms" in check and check[fastest + "_ms"] < check["per_wave_ms"]:
        select(fastest)
        step_variants(fastest + "+fused_unrotation/", True)
        select("per_wave")
    w.fused_unrotation = False
    emit({"done": True})


# how the parent starts the child above (a test harness may put another interpreter line here)
CANDIDATE_COMMAND = [sys.executable, os.path.abspath(__file__)]


def candidates_from_child(args, timeout_s=150):
    """Runs `bench.py --candidates` with this run's sizes and returns its JSON lines (those it
    wrote before it ended, however it ended) and a note on how it ended.  The child gets two and a
    half minutes (it needs about one, most of it the import of torch): a run that prints nothing
    for longer than that looks hung from outside."""
    import subprocess
    cmd = CANDIDATE_COMMAND + ["--candidates", "--steps", str(args.steps), "--warmup", str(args.warmup),
                               "--batch", str(args.batch)]
    for flag, on in (("--no-graph", args.no_graph), ("--serial-only", args.serial_only),
                     ("--no-autotune", args.no_autotune)):
        if on:
            cmd.append(flag)
    note = None
    print("bench.py: timing the other step variants in a child process ...", file=sys.stderr, flush=True)
    try:
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                           timeout=timeout_s)
        text = p.stdout
        if p.returncode != 0:
            note = "ended with status %d: %s" % (p.returncode, p.stderr.strip()[-200:])
    except subprocess.TimeoutExpired as e:          # (run() has ended the child by then)
        text = e.stdout if isinstance(e.stdout, str) else (e.stdout or b"").decode("utf-8", "replace")
        note = "stopped after %d s" % timeout_s
    except OSError as e:
        text, note = "", repr(e)[:200]
    lines = []
    for l in text.splitlines():
        try:
            d = json.loads(l)
        except ValueError:
            continue
        if isinstance(d, dict):
            lines.append(d)
    if note is None and not any(d.get("done") for d in lines):
        note = "ended before its last line"
    return lines, note


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the other workloads (sparse upstream gradient, vector types at "
                         "28x96^3, resampling), which are measured after the timed steps")
    ap.add_argument("--no-write-stream", action="store_true",
                    help="skip the forward call with every atom ignored (the write stream alone) "
                         "and the plain fill: for profiling runs, whose per-kernel means then "
                         "cover the real calls only")
    ap.add_argument("--small-extras", action="store_true",
                    help="cut the vector-type workloads down to 2 x 300 atoms: for dry runs of this "
                         "script (an emulated device), not for figures")
    ap.add_argument("--no-candidates", action="store_true",
                    help="time only the step in the reference's order, launch by launch, with the "
                         "library's default write-out (no child process): for profiling runs")
    ap.add_argument("--no-graph", action="store_true",
                    help="candidates: do not time the step as a captured HIP graph")
    ap.add_argument("--serial-only", action="store_true",
                    help="candidates: only the step in the reference's order on one stream")
    ap.add_argument("--no-autotune", action="store_true",
                    help="candidates: only the library's default write-out of the splat launch")
    ap.add_argument("--candidates", action="store_true",
                    help="(the child process that bench.py starts by itself) time the other ways of "
                         "enqueueing a step and the other write-out; one JSON line each")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library runs on one GPU (examples are independent; a larger job "
              "splits the batch over processes with no exchange) -- use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import libmolgrid_amd as mg
    import synth

    if not torch.cuda.is_available():
        print("bench.py: no ROCm device visible", file=sys.stderr)
        sys.exit(1)
    if args.candidates:
        run_candidates(args)
        return
    torch.cuda.set_device(0)

    w = Workload(args)
    B, T, D, cfg, gm, n_atoms = w.B, w.T, w.D, w.cfg, w.gm, w.n_atoms
    offsets, centers, moved, types, radii = w.offsets, w.centers, w.moved, w.types, w.radii
    grid, diff, grads = w.grid, w.diff, w.grads
    k_transform, k_forward, k_backward, k_unrotate = w.k_transform, w.k_forward, w.k_backward, w.k_unrotate
    k_backward_unrotated = w.k_backward_unrotated

    # The step in the reference's order, launch by launch, with the library's defaults: W warm-up
    # steps, then exactly K timed ones.  (The other ways of enqueueing a step are timed by a child
    # process at the end, see run_candidates.)
    variants = {"serial_eager": w.timed(w.step_serial)}
    w.step_serial()                               # the grids and gradients of a step again

    # per-kernel durations (events on the launch stream)
    it = max(args.steps, 10)
    ms_fwd = event_ms(k_forward, it)
    ms_bwd = event_ms(k_backward, it)
    ms_tr = event_ms(k_transform, it)
    in_step = step_breakdown([k_transform, k_forward, k_backward, k_unrotate], it)
    ms_bwd_unrot = event_ms(k_backward_unrotated, it)
    # What the write stream alone costs on this box: the same forward call with every atom's type
    # set to "ignored" (the sort launch does its work and drops them, the splat launch stores
    # zeros in its usual pattern and order, with no arithmetic), and a plain fill of the tensor.
    ms_fwd_stores = ms_fill = None
    if not args.no_write_stream:
        types_none = torch.full_like(types, -1.0)
        ms_fwd_stores = event_ms(lambda: w.k_forward_no_atoms(types_none), it)
        ms_fill = event_ms(lambda: grid.zero_(), it)
        del types_none
        k_forward()                               # the grids of the step again

    grid_bytes = B * T * D ** 3 * 4
    fwd_bytes = grid_bytes + n_atoms * 20          # grid written once + coords/type/radius read
    bwd_bytes = grid_bytes + n_atoms * 20 + n_atoms * 12
    fwd_gbs = fwd_bytes / (ms_fwd * 1e-3) / 1e9
    bwd_gbs = bwd_bytes / (ms_bwd * 1e-3) / 1e9

    dominant_fwd = ms_fwd >= ms_bwd
    roofline = {
        # one forward call = sort_atoms_kernel + splat_sorted_kernel; the duration is that of both
        "kernel": "sort_atoms_kernel + splat_sorted_kernel (forward)" if dominant_fwd
                  else "backward_index_kernel",
        "write_out": "per_wave",          # of the splat launch (the library's default)
        "bound": "hbm",
        "achieved": round(fwd_gbs if dominant_fwd else bwd_gbs, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round((fwd_gbs if dominant_fwd else bwd_gbs) / HBM_PEAK_GBS, 4),
        "traffic": forward_traffic() if dominant_fwd else measured_traffic("backward_index_kernel"),
        "traffic_source": TRAFFIC_PROFILE + " (rocprofv3 counters of this command, not of this run)",
        "algorithmic_bytes_per_launch": fwd_bytes if dominant_fwd else bwd_bytes,
        "avg_launch_ms": round(ms_fwd if dominant_fwd else ms_bwd, 4),
        # measured in this run: the forward call with its arithmetic removed, and a plain fill
        "write_stream_alone": None if ms_fwd_stores is None else {
            "forward_call_all_atoms_ignored_ms": round(ms_fwd_stores, 4),
            "frac": round(fwd_bytes / (ms_fwd_stores * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "write_out": "per_wave",
            "torch_fill_ms": round(ms_fill, 4),
            "torch_fill_frac": round(grid_bytes / (ms_fill * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        # the same kernel between the other launches of the step (see step_breakdown)
        "in_step_ms": round(in_step[1] if dominant_fwd else in_step[2], 4),
        "in_step_frac": round((fwd_bytes / in_step[1] if dominant_fwd else bwd_bytes / in_step[2])
                              / 1e6 / HBM_PEAK_GBS, 4),
    }
    kernels = {
        "forward": {"ms": round(ms_fwd, 4), "in_step_ms": round(in_step[1], 4), "grids_per_s": round(B / (ms_fwd * 1e-3), 1),
                    "GBps": round(fwd_gbs, 1), "hbm_frac": round(fwd_gbs / HBM_PEAK_GBS, 4)},
        "backward": {"ms": round(ms_bwd, 4), "in_step_ms": round(in_step[2], 4),
                     "unrotated_ms": round(ms_bwd_unrot, 4),
                     "atom_grads_per_s": round(n_atoms / (ms_bwd * 1e-3), 1),
                     "GBps": round(bwd_gbs, 1), "hbm_frac": round(bwd_gbs / HBM_PEAK_GBS, 4)},
        "transform": {"ms": round(ms_tr, 4), "in_step_ms": round(in_step[0], 4),
                      "unrotate_in_step_ms": round(in_step[3], 4)},
    }

    parity = None
    if not args.no_cpu:
        # the step once more, gradients before their un-rotation, against the oracle
        k_transform()
        k_forward()
        k_backward()
        torch.cuda.synchronize()
        parity = parity_sample(cfg, (0.5, 23.5), T, min(B, 5), moved, grid, diff, grads)

    if not args.no_extras:
        kernels.update(other_workloads(mg, synth, gm, offsets, centers, moved, types, radii, grid,
                                       diff, grads, n_atoms, bwd_bytes, small=args.small_extras))

    cpu = None
    if not args.no_cpu:
        nsample = B
        passes = 10            # about 10 s of single-thread work
        runs = [cpu_baseline(cfg, T, nsample, 1) for _ in range(passes)]
        r1 = {k: sum(r[k] for r in runs) for k in ("total_s", "forward_s", "backward_s")}
        r1["atoms"] = runs[0]["atoms"]
        cpu = {
            "value": round(passes * nsample / r1["total_s"], 2),
            "unit": "grids/s",
            "cores": 1,
            "kind": "port",
            "sample": "%d passes over the %d examples (%d atoms), transform + forward + backward + "
                      "gradient un-rotation, single thread like the reference's host loop"
                      % (passes, nsample, r1["atoms"]),
            "forward_grids_per_s": round(passes * nsample / r1["forward_s"], 2),
            "backward_atom_grads_per_s": round(passes * r1["atoms"] / r1["backward_s"], 1),
        }
        try:
            # resampling (configuration 4) on the CPU: a few grids, single thread
            import oracle
            import synth as _synth
            nint = 16
            rng = np.random.default_rng(4)
            src = rng.standard_normal((nint, T, D, D, D)).astype(np.float32)
            zeros = np.zeros((nint, 3), np.float32)
            t0 = time.perf_counter()
            oracle.interpolate_batch(0.5, 23.5, 0.5, 23.5, zeros, src,
                                     _synth.random_quaternions(rng, nint), zeros,
                                     rng.uniform(-1.5, 1.5, (nint, 3)).astype(np.float32), zeros,
                                     nthreads=1)
            cpu["interpolated_grids_per_s"] = round(nint / (time.perf_counter() - t0), 2)
            del src
        except Exception as e:  # pragma: no cover
            cpu["interpolated_grids_per_s"] = {"error": str(e)}
        try:
            import oracle
            nt = min(oracle.max_threads(), 16)
            if nt > 1:
                rn = cpu_baseline(cfg, T, B, nt)
                rn = cpu_baseline(cfg, T, B, nt)     # second pass: threads and pages are warm
                cpu["all_cores"] = {"value": round(B / rn["total_s"], 2), "cores": nt,
                                    "sample": "the %d examples, OpenMP over the batch" % B}
        except Exception as e:  # pragma: no cover
            cpu["all_cores"] = {"error": str(e)}

    # The other ways of enqueueing a step and the other write-out, from a child process started
    # now that this process has measured everything above (its results cannot be touched by what
    # the child does; the device is idle while the child runs).
    write_out = None
    child_note = None
    if not args.no_candidates:
        lines, child_note = candidates_from_child(args)
        for d in lines:
            if "candidate" in d:
                name = d["candidate"]
                if "error" in d:
                    variants[name + "_error"] = d["error"]
                else:
                    variants[name] = (d["ms_per_step"], d["enqueue_ms_per_step"])
            elif "write_out_check" in d:
                write_out = d["write_out_check"]
    timings = {k: v for k, v in variants.items() if isinstance(v, tuple)}
    best = min(timings, key=lambda k: timings[k][0])
    ms_per_step, enqueue_ms_per_step = timings[best]
    step_variants = {k: ({"ms_per_step": round(v[0], 4), "enqueue_ms_per_step": round(v[1], 4)}
                         if isinstance(v, tuple) else v) for k, v in variants.items()}
    if child_note is not None:
        step_variants["candidates_note"] = child_note
    if write_out is not None:
        used = best.split("/")[0].split("+")[0] if "/" in best else "per_wave"
        if used == "fused_unrotation":
            used = "per_wave"
        write_out["used"] = used
        if used != "per_wave" and dominant_fwd and (used + "_ms") in write_out:
            # `value` is from a step whose splat launch is another instance of the kernel (same grids
            # bit for bit, timed in the child with the same events): the headline figures of this
            # object are that call's, the default's move aside (the committed counter summary covers
            # the default only, so no measured traffic for this one)
            ms_used = write_out[used + "_ms"]
            gbs = fwd_bytes / (ms_used * 1e-3) / 1e9
            roofline["per_wave_write_out"] = {k: roofline[k] for k in
                                              ("avg_launch_ms", "achieved", "frac", "traffic")}
            roofline.update(avg_launch_ms=ms_used, achieved=round(gbs, 1),
                            frac=round(gbs / HBM_PEAK_GBS, 4), traffic=None)
            roofline["write_out"] = used

    out = {
        "metric": "grids/sec, 28x48^3 fp32 batch 50, fwd + atom-grad bwd; % of HBM roofline",
        "value": round(B / (ms_per_step * 1e-3), 1),
        "unit": "grids/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        # which way of enqueueing the step `value` is from (step_variants lists all of them):
        # serial = the reference's order on one stream, overlapped = the sort launch beside the
        # backward pass; eager = launch by launch, graph = one captured HIP graph; a prefix such as
        # "paged/" = with that instance of the splat launch (forward_write_out lists them),
        # "fused_unrotation" = the gradients' un-rotation inside the backward launch
        "launch": best,
        "ms_per_step": round(ms_per_step, 4),
        # wall time the host needs to enqueue a step (the timed loop before its synchronize): when
        # this comes close to ms_per_step the loop is bound by the host, not by the kernels
        "enqueue_ms_per_step": round(enqueue_ms_per_step, 4),
        "step_variants": step_variants,
        "forward_write_out": write_out,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]+[2]: batch %d ragged complexes (%d atoms), random "
                               "rotation + translation, 28x48^3 grid at 0.5 A, Gaussian density; "
                               "transform + forward + atom-gradient backward + un-rotation"
                               % (B, n_atoms),
                   "batch": B, "atoms": n_atoms, "grid": [T, D, D, D]},
        "roofline": roofline,
        "kernels": kernels,
        "parity": parity,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
