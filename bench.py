"""Benchmark of the energy / force / virial hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

A step is one pass of the hot path over one batch of synthetic input resident in HBM.  The
default workload is the configuration the headline target is quoted on (1,048,576-atom NEP
molecular-dynamics step: neighbour-list rebuild + descriptors + per-species network + force /
virial); the other workloads are the remaining benchmark configurations.  Prints one JSON
line (metric: atom-steps/s) with a `roofline` object for the kernel that takes the most time
and a `cpu_baseline` object (the reference's CPU code compiled into oracle/_ref when present,
else this repository's CPU restatement) timed on the host cores on a bounded sample.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
PEAK_FP32_TFLOPS = 157.3       # MI355X fp32
PEAK_FP64_TFLOPS = 78.6        # MI355X fp64


# ------------------------------------------------------------------------------------------------
# algorithmic work (FMA = 2 flops), per centre atom
# ------------------------------------------------------------------------------------------------
def nep_flops_per_atom(nr_mean, na_mean, K=8, n_r=6, n_a=4, D=22, H=50):
    """Factored NEP E/F/V: per radial neighbour 14 + c(K) + 4K n_r + 3 n_r, per angular neighbour
    c(K) + 4K n_a + 210 + 480 n_a, per atom 144 n_a + 4 D H + 15 H, with c(K) = 14K + 24."""
    cK = 14 * K + 24
    return (nr_mean * (14 + cK + 4 * K * n_r + 3 * n_r) +
            na_mean * (cK + 4 * K * n_a + 210 + 48 * n_a + 432 * n_a) + 144 * n_a + 4 * D * H + 15 * H)


def nep_efv_bytes_per_atom(nr_mean, s):
    """E/F/V operator, algorithmic bytes per atom: ilist / numneigh / type (12), the valid part of the
    row (index + relative vector per neighbour), the neighbour-type gather (4 per neighbour) and the
    force written (3 s)."""
    return 12 + nr_mean * (4 + 3 * s) + 4 * nr_mean + 3 * s


def nbl_bytes_per_atom(nr_mean, s, umax, in_place):
    """Neighbour list, algorithmic bytes per atom.  Fresh build: position + type in, ilist / numneigh /
    types and the full padded rows out.  In-place update (the calculator's steady state): a row is
    written as far as its old or new length reaches, rounded up to four slots."""
    if in_place:
        return (3 * s + 4) + 12 + (nr_mean + 2) * (4 + 3 * s)
    return (3 * s + 4) + 12 + umax * (4 + 3 * s)


def mtp_flops_per_atom(nn_mean, K, nmus, kmax, n_basic, n_times, n_scalar):
    """Linear-MTP E/F/V: per neighbour 8 + 8K + 30 + 4K nmus + 4 kmax + 29 n_basic, per atom
    9 n_times + 4 n_scalar."""
    return nn_mean * (8 + 8 * K + 30 + 4 * K * nmus + 4 * kmax + 29 * n_basic) + 9 * n_times + 4 * n_scalar


def mtp_loss_flops_per_atom(nn_mean, K, nmus, kmax, n_basic, n_times, n_scalar):
    """Training step (E/F/V + loss gradient): F_efv + per neighbour 2 (8K + 30 + 4 kmax + 4K nmus)
    + 70 n_basic, per atom 24 n_times + 6 n_scalar."""
    return (mtp_flops_per_atom(nn_mean, K, nmus, kmax, n_basic, n_times, n_scalar) +
            nn_mean * (2 * (8 * K + 30 + 4 * kmax + 4 * K * nmus) + 70 * n_basic) + 24 * n_times + 6 * n_scalar)


def profile_report(L):
    from ai2pot_amd import _lib
    buf = ctypes.create_string_buffer(1 << 16)
    _lib.check(L.a2p_profile_report(buf, ctypes.c_size_t(len(buf))))
    kernels = {}
    for line in buf.value.decode().splitlines():
        name, count, ms = line.split()
        kernels[name] = dict(launches=int(count), total_ms=float(ms), avg_ms=float(ms) / int(count))
    return kernels


def timed(step, steps, warmup, L, keep=2):
    """Times `steps` steps after `warmup` untimed ones.  Every launch of the library is bracketed by
    HIP events during the warm-up steps, which gives the per-kernel breakdown; in the timed region
    only the `keep` longest kernels stay bracketed (two events per launch cost the step about 3 % at
    fifteen launches), and their figures are the timed region's."""
    import torch
    L.a2p_profile_select(None)
    L.a2p_profile_enable(0)
    plain = 1 if warmup > 1 else 0          # the very first step carries one-time costs (code loading)
    for k in range(plain):
        step(k)
    torch.cuda.synchronize()
    L.a2p_profile_enable(1 if warmup > 0 else 0)
    for k in range(plain, warmup):
        step(k)
    torch.cuda.synchronize()
    kernels = {}
    if warmup > 0:
        kernels = profile_report(L)
        for v in kernels.values():
            v["per_step_ms"] = v["total_ms"] / (warmup - plain)
            v["measured_in"] = "warm-up"
        top = sorted(kernels, key=lambda k: -kernels[k]["total_ms"])[:keep]
        L.a2p_profile_select(",".join(top).encode())
    L.a2p_profile_enable(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        step(warmup + k)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for name, v in profile_report(L).items():
        v["per_step_ms"] = v["total_ms"] / steps
        v["measured_in"] = "timed region"
        kernels[name] = v
    L.a2p_profile_enable(0)
    L.a2p_profile_select(None)
    return t1 - t0, kernels


def timed_replay(replay, steps, warmup):
    """Wall time of `steps` replays of a captured step (no per-kernel events: a replay is one launch)."""
    import torch
    for _ in range(warmup):
        replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        replay()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


# Counter figures come from the rocprofv3 summaries under profiles/: a line
#     @data <workload> <kernel> fetch_kib=<FETCH_SIZE> write_kib=<WRITE_SIZE> flops_executed=<flops per launch>
# holds, per launch of one kernel, the raw FETCH_SIZE / WRITE_SIZE readings (KiB; scaled here by what the same
# counters read for a plain copy of known size: 2.00 and 1.00, `bench.py --workload hbm_copy_probe`) and the
# floating-point operations the kernel executed (2 x FMA + MUL + ADD instructions x 64 lanes).  Kernels without
# such a line report null.
FETCH_SCALE, WRITE_SCALE = 2.00, 1.00
_PROFILE_DATA = None


def profile_data():
    global _PROFILE_DATA
    if _PROFILE_DATA is None:
        _PROFILE_DATA = {}
        root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")
        for name in sorted(os.listdir(root)) if os.path.isdir(root) else []:
            if not name.endswith(".txt"):
                continue
            with open(os.path.join(root, name)) as f:
                for line in f:
                    if not line.startswith("@data "):
                        continue
                    parts = line.split()
                    rec = _PROFILE_DATA.setdefault((parts[1], parts[2]), {})
                    for kv in parts[3:]:
                        k, v = kv.split("=")
                        rec[k] = float(v)
    return _PROFILE_DATA


def measured_traffic(workload, kernel):
    rec = profile_data().get((workload, kernel), {})
    if "fetch_kib" not in rec or "write_kib" not in rec:
        return None
    return (FETCH_SCALE * rec["fetch_kib"] + WRITE_SCALE * rec["write_kib"]) * 1024.0


def executed_flops(workload, kernel):
    return profile_data().get((workload, kernel), {}).get("flops_executed")


def roofline_of(kernels, work, workload=None):
    """work: {label: (bound, amount per launch, unit, peak, scale, engine)}.  A label may name several
    kernels joined by '+': they form one operator, whose duration per launch is the sum of the
    kernels' average durations.  Returns the entry of the label with the largest time (with `traffic`
    when profiles/ holds a counter run for it) and the list of all entries."""
    def entry(label):
        names = label.split("+")
        if not all(nm in kernels for nm in names):
            return None
        bound, amount, unit, peak, scale, engine = work[label]
        avg_ms = sum(kernels[nm]["avg_ms"] for nm in names)
        achieved = amount / (avg_ms * 1e-3) / scale
        traffic = [measured_traffic(workload, nm) for nm in names]
        e = dict(kernel=label, bound=bound, achieved=achieved, peak=peak, unit=unit, frac=achieved / peak,
                 traffic=sum(traffic) if all(t is not None for t in traffic) else None, avg_ms=avg_ms,
                 engine=engine, amount_per_launch=amount)
        if bound == "valu":
            # what the kernels executed (counter run under profiles/) beside the algorithmic count above
            ex = [executed_flops(workload, nm) for nm in names]
            if all(x is not None for x in ex):
                e["executed"] = sum(ex) / (avg_ms * 1e-3) / scale
                e["executed_frac"] = e["executed"] / peak
                e["executed_per_launch"] = sum(ex)
            else:
                e["executed"] = None
        return e
    entries = [e for e in (entry(l) for l in work) if e is not None]
    if not entries:
        return None, []
    return max(entries, key=lambda e: e["avg_ms"]), entries


# ------------------------------------------------------------------------------------------------
# NEP molecular-dynamics step (configurations 2 and 5)
# ------------------------------------------------------------------------------------------------
def nep_structure(kind, n_or_reps):
    from ai2pot_amd import synth
    if kind == "fcc":
        a = 316.7 / 64.0                      # 0.033 atoms / A^3
        lattice, pos = synth.fcc_cell(n_or_reps, a, 0.15, 1006)
        seed = 2006
    else:                                     # configuration 2: random packing, d_min 2.2
        L = (n_or_reps / 0.033) ** (1.0 / 3.0)
        lattice, pos = synth.random_packed(n_or_reps, [L, L, L], 2.2, 1003)
        seed = 2003
    types = synth.rng_randint(seed, pos.shape[0], 3)
    disp = synth.rng_normal(5006, pos.size, 0.0, 0.01).reshape(-1, 3)
    return lattice, pos, types, disp


class OpsStepper:
    """The molecular-dynamics step through registered operators only (torch.ops.nblist.find_info4mlff_compact_
    + torch.ops.nep.nepToEFVCompactOp from the bind libraries), as a TorchScript model or a C++ host would
    drive it: no ctypes, no calculator object.  Validation is switched off for the timed loop (no
    synchronisation per call) and the status word is read once at the end."""

    def __init__(self, model, n, lattice, types, dev, umax=200, reorder_every=64):
        import torch
        from ai2pot_amd import bind_build
        for name in ("libnblist_bind.so", "libnep_bind.so"):
            path = os.path.join(os.path.dirname(os.path.abspath(bind_build.__file__)), "_lib", name)
            if not os.path.exists(path):
                sys.exit("bench.py: %s missing: run python -m ai2pot_amd.build --bind" % path)
            torch.ops.load_library(path)
        f = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(dev)
        self.model_args = (int(model["chebyshev_size"]), int(model["n_radial_basis"]), int(model["n_angular_basis"]),
                           int(model["l_max"]), f(model["coeffs"]), f(model["w0"]), f(model["b0"]), f(model["w1"]),
                           f(model["type_bias"]))
        self.tail = (torch.from_numpy(np.ascontiguousarray(model["type_map"], np.int32)).to(dev),
                     float(model["rmax_radial"]), float(model["rmax_angular"]), f(model["q_scaler"]))
        self.rr, self.ra = float(model["rmax_radial"]), float(model["rmax_angular"])
        self.lattice = torch.from_numpy(np.ascontiguousarray(lattice, np.float32).reshape(3, 3))
        self.types = torch.from_numpy(np.ascontiguousarray(types, np.int32)).to(dev)
        self.n, self.umax, self.reorder_every = n, umax, reorder_every
        i32 = dict(dtype=torch.int32, device=dev)
        self.rows = [torch.empty(n, **i32), torch.empty(n, **i32), torch.empty((n, umax), **i32),
                     torch.empty((n, umax, 3), dtype=torch.float32, device=dev), torch.empty(n, **i32)]
        self.compact = torch.empty(torch.ops.nblist.compact_bytes(n, umax, 4), dtype=torch.uint8, device=dev)
        self.builds = 0
        self.build = torch.ops.nblist.find_info4mlff_compact_
        self.efv = torch.ops.nep.nepToEFVCompactOp

    def step(self, coords):
        update = (1 if self.builds else 0) | (2 if self.builds % self.reorder_every else 0)
        self.build(self.lattice, self.types, coords, self.rr, self.umax, True, [True, True, True], self.rr, self.ra,
                   update, *self.rows, self.compact)
        self.builds += 1
        return self.efv(*self.model_args, self.types, self.compact, self.umax, *self.tail)


def run_nep_md(args, kind, size, rebuild=True, via_ops=False):
    import torch
    from ai2pot_amd import _lib, synth
    from ai2pot_amd.calculator import NepCalculator
    dev = torch.device("cuda:0")
    lattice, pos, types, disp = nep_structure(kind, size)
    n = pos.shape[0]
    model = synth.nep_model(seed=3006)
    # rebuilds after the first size their bin grid from the first one's bound: no host synchronisation in the step
    calc = NepCalculator(model, n, lattice, types, umax=200, dtype=torch.float32, device=dev, sync_free=rebuild)
    ops_path = OpsStepper(model, n, lattice, types, dev) if (via_ops or (rebuild and calc.path == "gather" and not args.no_other_configs)) else None
    coords0 = torch.from_numpy(pos.astype(np.float32)).to(dev)
    disp_t = torch.from_numpy(disp.astype(np.float32)).to(dev)
    coords = torch.empty_like(coords0)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    calc.rebuild(coords0, stream)

    def step(k):
        if rebuild:     # a small deterministic displacement: every step builds a different list
            torch.add(coords0, disp_t, alpha=float(np.sin(0.37 * k)), out=coords)
            return ops_path.step(coords) if via_ops else calc.step(coords)
        calc.evaluate(stream)

    L = _lib.lib()
    if via_ops:
        torch.ops.nblist.set_validate(False)
        torch.ops.nep.set_validate(False)
        ops_path.step(coords0)                       # a synchronised build first: it sets the bound
        torch.ops.nblist.set_sync_free(True)
    elapsed, kernels = timed(step, args.steps, args.warmup, L, keep=3)
    if via_ops:
        last = step(args.warmup + args.steps - 1)
        ref = calc.step(coords)
        torch.ops.nblist.check_status(coords)
        torch.ops.nblist.set_sync_free(False)
        torch.ops.nblist.set_validate(True)
        torch.ops.nep.set_validate(True)
        # same kernels; the processing orders of the two drivers may differ, hence rounding-level bars
        if not (torch.allclose(last[0], ref[0], rtol=1e-5) and torch.allclose(last[1][0], ref[1], rtol=1e-4, atol=1e-4)
                and torch.allclose(last[2][0], ref[2], rtol=1e-4, atol=1e-2)):
            sys.exit("bench.py: the operator path and the calculator disagree")
    if args.graph:
        # the whole step (coordinate update, sync-free rebuild, E/F/V) as one HIP graph
        graph = torch.cuda.CUDAGraph()
        alpha = torch.zeros((), dtype=torch.float32, device=dev)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                # one call on a capture-capable stream first
            if rebuild:
                calc.step(coords)
            else:
                calc.evaluate(ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            if rebuild:
                torch.addcmul(coords0, disp_t, alpha, out=coords)
                calc.step(coords)
            else:
                calc.evaluate(ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        state = {"k": 0}

        def replay():
            if rebuild:
                alpha.fill_(float(np.sin(0.37 * state["k"])))
                state["k"] += 1
            graph.replay()
        elapsed = timed_replay(replay, args.steps, args.warmup)
    calc.check()
    if not np.isfinite(float(calc.etot.item())):
        sys.exit("bench.py: non-finite energy")
    order_refresh = None
    if rebuild and calc.path == "gather" and not via_ops:
        # The processing order of the atoms (a locality hint) is renewed every calc.reorder_every rebuilds: the timed
        # region holds such a rebuild whenever it spans a multiple of that count.  Its cost, measured on its own:
        def rebuild_ms(refresh, reps=6):
            best = None
            for _ in range(reps):
                calc._builds = calc.reorder_every if refresh else 1
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                calc.rebuild(coords, stream)
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t0) * 1e3
                best = dt if best is None else min(best, dt)
            return best
        kept, fresh = rebuild_ms(False), rebuild_ms(True)
        first, last = args.warmup + 1, args.warmup + args.steps        # the calculator's build counter in the timed region
        inside = last // calc.reorder_every - (first - 1) // calc.reorder_every
        order_refresh = dict(reorder_every=calc.reorder_every, rebuild_ms_order_kept=kept, rebuild_ms_order_renewed=fresh,
                             amortised_ms_per_step=(fresh - kept) / calc.reorder_every,
                             renewals_inside_timed_region=inside)
    nn_r = float(calc.numneigh.float().mean().item())
    r = calc.rcs.norm(dim=2)
    nn_a = float(((r > 0) & (r <= model["rmax_angular"])).sum().item()) / n
    s = 4
    flops = nep_flops_per_atom(nn_r, nn_a) * n
    efv_bytes = nep_efv_bytes_per_atom(nn_r, s) * n
    valu = ("valu", flops, "TFLOP/s", PEAK_FP32_TFLOPS, 1e12, "valu_fp32")
    work = {
        # the energy / force / virial operator as a whole, against the fp32 vector peak: whichever kernels serve it
        "nep_adjoint_kernel+nep_gather_kernel": valu,
        "nep_stage_kernel+nep_staged_kernel+reduce_sum": valu,
        "nep_group_kernel+reduce_sum": valu,
        "nep_efv_kernel": valu,
        "nbl_lists": ("hbm", nbl_bytes_per_atom(nn_r, s, 200, rebuild) * n, "GB/s", PEAK_HBM_GBS, 1e9, "hbm"),
    }
    config = {"workload": args.workload, "natoms": n, "species": 3,
              "model": "NEP radial+3-body K=8 n_r=6 n_a=4 l_max=4 H=50", "rcut_radial": 7.0, "rcut_angular": 4.0,
              "umax": 200, "mean_neighbors_radial": nn_r, "mean_neighbors_angular": nn_a,
              "per_step": ("neighbor rebuild (padded arrays + compact lists) + " if rebuild else "") +
                          "descriptors + ANN + force/virial",
              "path": calc.path, "launch": "hip graph replay" if args.graph else "eager",
              "driver": "torch.ops.nblist.find_info4mlff_compact_ + torch.ops.nep.nepToEFVCompactOp, validation off"
                        if via_ops else "NepCalculator (ctypes over the C ABI)"}
    roof, entries = roofline_of(kernels, work, args.workload)
    if roof is not None and roof["bound"] == "valu":
        # the same operator against the memory roofline (algorithmic bytes of the E/F/V operator)
        gbs = efv_bytes / (roof["avg_ms"] * 1e-3) / 1e9
        roof["hbm"] = dict(achieved=gbs, peak=PEAK_HBM_GBS, unit="GB/s", frac=gbs / PEAK_HBM_GBS, amount_per_launch=efv_bytes)
    extra = {"rooflines": entries}
    if order_refresh is not None:
        extra["order_refresh"] = order_refresh
        config["reorder_every"] = calc.reorder_every
    if rebuild and calc.path == "gather" and not args.graph and not args.no_other_configs:
        # the same step without the padded firstneigh / rcs arrays (energy, forces and virial only)
        lean = NepCalculator(model, n, lattice, types, umax=200, dtype=torch.float32, device=dev, padded=False,
                             sync_free=True)
        lean.rebuild(coords0, stream)

        def lean_step(k):
            torch.add(coords0, disp_t, alpha=float(np.sin(0.37 * k)), out=coords)
            return lean.step(coords)
        for k in range(args.warmup):
            lean_step(k)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(args.steps):
            lean_step(args.warmup + k)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        lean.check()
        extra["without_padded_arrays"] = dict(ms_per_step=dt * 1e3 / args.steps, value=n * args.steps / dt,
                                              unit="atom-steps/s")
        del lean
        # the headline step (padded arrays included) with the atoms processed in the order they are given in
        # instead of along the library's space-filling curve: the synthetic crystal is written cell by cell
        inorder = NepCalculator(model, n, lattice, types, umax=200, dtype=torch.float32, device=dev, sync_free=True,
                                reorder_every=0)
        inorder.rebuild(coords0, stream)

        def inorder_step(k):
            torch.add(coords0, disp_t, alpha=float(np.sin(0.37 * k)), out=coords)
            return inorder.step(coords)
        for k in range(args.warmup):
            inorder_step(k)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(args.steps):
            inorder_step(args.warmup + k)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        inorder.check()
        extra["atoms_processed_in_input_order"] = dict(ms_per_step=dt * 1e3 / args.steps, value=n * args.steps / dt,
                                                       unit="atom-steps/s")
        del inorder
        if not via_ops:
            # the same step (padded arrays included) driven through the registered operators alone
            torch.ops.nblist.set_validate(False)
            torch.ops.nep.set_validate(False)
            ops_path.step(coords0)                   # a synchronised build first: it sets the bound
            torch.ops.nblist.set_sync_free(True)

            def ops_step(k):
                torch.add(coords0, disp_t, alpha=float(np.sin(0.37 * k)), out=coords)
                return ops_path.step(coords)
            for k in range(args.warmup):
                ops_step(k)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for k in range(args.steps):
                ops_step(args.warmup + k)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            torch.ops.nblist.check_status(coords)
            torch.ops.nblist.set_sync_free(False)
            torch.ops.nblist.set_validate(True)
            torch.ops.nep.set_validate(True)
            extra["through_torch_ops"] = dict(ms_per_step=dt * 1e3 / args.steps, value=n * args.steps / dt,
                                              unit="atom-steps/s", vs_calculator=dt / elapsed)
    return n, elapsed, kernels, roof, config, "f32", extra


def cpu_baseline_nep(sample_reps=32, repeats=2):
    """131072-atom sample of the same recipe: single-threaded list + OpenMP E/F/V, as the reference."""
    import oracle
    from ai2pot_amd import synth
    lattice, pos, types, _ = nep_structure("fcc", sample_reps)
    m = synth.nep_model(seed=3006)
    use_ref = oracle.ref_available("nep") and oracle.ref_available("nblist")
    nbl = oracle.ref_nblist if use_ref else oracle.nblist
    efv = oracle.ref_nep_efv if use_ref else oracle.nep_efv
    n = pos.shape[0]
    best = None
    for _ in range(repeats):
        t0 = time.time()
        out = nbl(lattice.astype(np.float32), types, pos.astype(np.float32), 7.0, 200)
        efv(m, synth.pack_batch([out]), np.float32)
        dt = time.time() - t0
        best = dt if best is None else min(best, dt)
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return dict(value=n / best, unit="atom-steps/s", cores=threads, kind="reference" if use_ref else "port",
                sample="%d atoms (FCC %d^3 x 4, same recipe), list rebuild (1 thread) + NEP E/F/V (OpenMP, "
                       "%d threads), best of %d" % (n, sample_reps, threads, repeats))


# ------------------------------------------------------------------------------------------------
# linear MTP (configurations 1, 3, 4)
# ------------------------------------------------------------------------------------------------
def mtp_setup(cfg):
    """Structures, lists (built on the GPU once, outside the timed region) and model of a config."""
    import torch
    from ai2pot_amd import mtp_param, nblist, synth
    dev = torch.device("cuda:0")
    if cfg == 1:
        lat, pos = synth.diamond_cell()
        structs = [(lat, pos, np.zeros(216, np.int32))]
        level, nt, K, rmax, rmin, lohi, seed = 10, 1, 8, 5.0, 0.5, (-0.1, 0.1), 3001
    elif cfg == 3:
        lat, pos = synth.random_packed(8192, [64.0, 51.2, 50.0], 2.0, 1004)
        structs = [(lat, pos, synth.rng_randint(2004, 8192, 4))]
        level, nt, K, rmax, rmin, lohi, seed = 20, 4, 10, 5.5, 1.8, (-0.05, 0.05), 3004
    else:
        rho = synth.rng_uniform(1005, 64, 0.03, 0.05)
        structs = []
        for b in range(64):
            Lb = (128.0 / rho[b]) ** (1.0 / 3.0)
            lat, pos = synth.random_packed(128, [Lb, Lb, Lb], 2.0, 11005 + b)
            structs.append((lat, pos, synth.rng_randint(21005 + b, 128, 3)))
        level, nt, K, rmax, rmin, lohi, seed = 16, 3, 8, 5.0, 0.0, None, 3005
    tables = mtp_param.mtp_param(level)
    if lohi is not None:
        m = synth.mtp_model(tables, nt, K, rmax, rmin, seed, lo=lohi[0], hi=lohi[1])
    else:   # the distributions of the reference's LinearMtp.__init__ (linear_mtp.py:74-88)
        m = synth.mtp_model(tables, nt, K, rmax, rmin, seed)
        S = m["linear_coeffs"].size
        m["coeffs"] = synth.rng_normal(seed, m["coeffs"].size, 0, 0.1) + synth.rng_uniform(seed + 7, m["coeffs"].size)
        m["linear_coeffs"] = synth.rng_normal(seed + 1, S, 0, np.sqrt(2.0 / (S + 1)))
        m["type_bias"] = synth.rng_normal(seed + 2, nt, 0, 1.0)
    lists = []
    for lat, pos, ty in structs:
        out = nblist.find_info4mlff_device(lat, torch.from_numpy(ty).to(dev), torch.from_numpy(pos).to(dev), rmax, 200)
        lists.append(tuple(o.cpu().numpy() if hasattr(o, "cpu") else o for o in out))
    nb = synth.pack_batch(lists)
    return m, nb, tables


def run_mtp(args, cfg):
    import torch
    from ai2pot_amd import _lib, ops, synth
    dev = torch.device("cuda:0")
    m, nb, tables = mtp_setup(cfg)
    f64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64)).to(dev)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)
    md = {k: f64(m[k]) for k in ("coeffs", "linear_coeffs", "type_bias", "q_scaler")}
    tb = {k: i32(m[k]) for k in ("alpha_index_basic", "alpha_index_times", "alpha_moment_mapping", "type_map")}
    d = {k: i32(nb[k]) for k in ("binum", "bilist", "bnumneigh", "bfirstneigh", "btypes")}
    d["brcs"] = f64(nb["brcs"])
    B, P = nb["bilist"].shape
    natoms = int(nb["binum"].sum())
    nn = float(nb["bnumneigh"].sum()) / natoms
    common = (m["chebyshev_size"], 1.0, md["coeffs"], md["linear_coeffs"], md["type_bias"],
              m["alpha_moments_count"], tb["alpha_index_basic"], tb["alpha_index_times"], tb["alpha_moment_mapping"],
              m["nmus"], d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"],
              tb["type_map"], 0, m["rmax"], m["rmin"], md["q_scaler"])
    kmax = int(tables["alpha_index_basic"][:, 1:].sum(1).max())
    sizes = (m["chebyshev_size"], m["nmus"], kmax, tables["alpha_index_basic"].shape[0],
             tables["alpha_index_times"].shape[0], tables["alpha_moment_mapping"].size)
    if cfg == 4:
        lab = (f64(synth.rng_normal(4005, B * P, -4.0, 0.2).reshape(B, P).sum(1)),
               f64(synth.rng_normal(4006, B * P * 3, 0.0, 1.0).reshape(B, P, 3)),
               f64(synth.rng_normal(4007, B * 9, 0.0, 0.5).reshape(B, 9)))
        out = {}

        def step(k):    # forward + analytic backward w.r.t. all parameters, as one training step
            out["r"] = ops.mtp_loss_step(1.0, 1.0, 1.0, lab[0], lab[1], lab[2], *common, want_grad=True,
                                         validate=False)
        flops = mtp_loss_flops_per_atom(nn, *sizes) * natoms
        label = "mtp_loss_bwd_kernel"
    else:
        def step(k):
            ops.linearMtpToEFVOp(*common, 0.0, 0.0, None, None, validate=False)
        flops = mtp_flops_per_atom(nn, *sizes) * natoms
        label = "mtp_efv_kernel"
    L = _lib.lib()
    elapsed, kernels = timed(step, args.steps, args.warmup, L)
    if args.graph:
        if cfg == 4:
            sys.exit("bench.py: --graph is wired for the energy / force / virial workloads")
        from ai2pot_amd.graph import GraphedCall
        g = GraphedCall(ops.linearMtpToEFVOp, *common, 0.0, 0.0, None, None)
        elapsed = timed_replay(g.replay, args.steps, args.warmup)
    _lib.check_status(torch.cuda.current_stream(dev).cuda_stream)
    work = {label: ("valu", flops if cfg != 4 else flops - mtp_flops_per_atom(nn, *sizes) * natoms, "TFLOP/s",
                    PEAK_FP64_TFLOPS, 1e12, "valu_fp64"),
            "mtp_efv_kernel": ("valu", mtp_flops_per_atom(nn, *sizes) * natoms, "TFLOP/s", PEAK_FP64_TFLOPS, 1e12,
                               "valu_fp64")}
    config = {"workload": args.workload, "natoms": natoms, "structures": B, "natoms_pad": P,
              "model": "linear MTP level %d K=%d" % ({1: 10, 3: 20, 4: 16}[cfg], m["chebyshev_size"]),
              "species": int(m["type_map"].size), "rmax": m["rmax"], "rmin": m["rmin"], "mean_neighbors": nn,
              "per_step": "loss forward + analytic gradient w.r.t. coeffs/linear/bias" if cfg == 4 else
                          "energy + force + virial (list built once, outside the timed region)",
              "launch": "hip graph replay" if args.graph else "eager"}
    roof, entries = roofline_of(kernels, work, args.workload)
    return natoms, elapsed, kernels, roof, config, "f64", {"rooflines": entries}


def run_nep_train(args):
    """NEP training step (the second model family's counterpart of configuration 4): the 64 x 128-atom
    structures of that configuration, fp32 (the reference trains NEP in single precision), loss forward
    + analytic gradient w.r.t. all parameters."""
    import torch
    from ai2pot_amd import _lib, nblist, ops, synth
    dev = torch.device("cuda:0")
    rho = synth.rng_uniform(1005, 64, 0.03, 0.05)
    lists = []
    for b in range(64):
        Lb = (128.0 / rho[b]) ** (1.0 / 3.0)
        lat, pos = synth.random_packed(128, [Lb, Lb, Lb], 2.0, 11005 + b)
        ty = synth.rng_randint(21005 + b, 128, 3)
        out = nblist.find_info4mlff_device(lat, torch.from_numpy(ty).to(dev), torch.from_numpy(pos).to(dev), 6.0, 200)
        lists.append(tuple(o.cpu().numpy() if hasattr(o, "cpu") else o for o in out))
    nb = synth.pack_batch(lists)
    m = synth.nep_model(seed=3007, rmax_radial=6.0, rmax_angular=4.0)
    f32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(dev)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)
    md = {k: f32(m[k]) for k in ("coeffs", "w0", "b0", "w1", "type_bias", "q_scaler")}
    d = {k: i32(nb[k]) for k in ("binum", "bilist", "bnumneigh", "bfirstneigh", "btypes")}
    d["brcs"] = f32(nb["brcs"])
    B, P = nb["bilist"].shape
    natoms = int(nb["binum"].sum())
    nn = float(nb["bnumneigh"].sum()) / natoms
    r = np.linalg.norm(nb["brcs"], axis=3)
    nn_a = float(((r > 0) & (r <= m["rmax_angular"])).sum()) / natoms
    lab = (f32(synth.rng_normal(4005, B * P, -4.0, 0.2).reshape(B, P).sum(1)),
           f32(synth.rng_normal(4006, B * P * 3, 0.0, 1.0).reshape(B, P, 3)),
           f32(synth.rng_normal(4007, B * 9, 0.0, 0.5).reshape(B, 9)))
    tm = i32(m["type_map"])

    def step(k):
        ops.nep_loss_step(1.0, 1.0, 1.0, lab[0], lab[1], lab[2], m["chebyshev_size"], m["n_radial_basis"],
                          m["n_angular_basis"], m["l_max"], md["coeffs"], md["w0"], md["b0"], md["w1"], md["type_bias"],
                          d["binum"], d["bilist"], d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"], tm, 0,
                          m["rmax_radial"], m["rmax_angular"], md["q_scaler"], want_grad=True, validate=False)
    L = _lib.lib()
    elapsed, kernels = timed(step, args.steps, args.warmup, L)
    _lib.check_status(torch.cuda.current_stream(dev).cuda_stream)
    # the gradient pass repeats the descriptor work with tangents (x2) and adds the outer products of the
    # hidden layer (4 D H) and the two coefficient-gradient contractions: counted as 2.5 x the E/F/V flops
    work = {"nep_loss_bwd_kernel": ("valu", 2.5 * nep_flops_per_atom(nn, nn_a) * natoms, "TFLOP/s", PEAK_FP32_TFLOPS,
                                    1e12, "valu_fp32")}
    config = {"workload": args.workload, "natoms": natoms, "structures": B, "natoms_pad": P, "species": 3,
              "model": "NEP radial+3-body K=8 n_r=6 n_a=4 l_max=4 H=50", "rcut_radial": 6.0, "rcut_angular": 4.0,
              "mean_neighbors_radial": nn, "mean_neighbors_angular": nn_a,
              "per_step": "E/F/V + loss forward + analytic gradient w.r.t. coeffs/w0/b0/w1/bias"}
    roof, entries = roofline_of(kernels, work, args.workload)
    return natoms, elapsed, kernels, roof, config, "f32", {"rooflines": entries}


def run_mtp_solver(args):
    """The normal equations of the linear parameters (LinMatrixLinVectorOp) on configuration 4's structures, level
    16: the components of all 92 scalar moments from one pass over the atoms, plus three Gram products by the BLAS."""
    import torch
    from ai2pot_amd import _lib, ops, synth
    dev = torch.device("cuda:0")
    m, nb, tables = mtp_setup(4)
    f64 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64)).to(dev)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)
    md = {k: f64(m[k]) for k in ("coeffs", "linear_coeffs", "type_bias", "q_scaler")}
    tb = {k: i32(m[k]) for k in ("alpha_index_basic", "alpha_index_times", "alpha_moment_mapping", "type_map")}
    d = {k: i32(nb[k]) for k in ("binum", "bilist", "bnumneigh", "bfirstneigh", "btypes")}
    d["brcs"] = f64(nb["brcs"])
    B, P = nb["bilist"].shape
    natoms = int(nb["binum"].sum())
    lab = (f64(synth.rng_normal(4005, B * P, -4.0, 0.2).reshape(B, P).sum(1)),
           f64(synth.rng_normal(4006, B * P * 3, 0.0, 1.0).reshape(B, P, 3)),
           f64(synth.rng_normal(4007, B * 9, 0.0, 0.5).reshape(B, 9)))

    def step(k):
        ops.LinMatrixLinVectorOp(1.0, 1.0, 1.0, lab[0], lab[1], lab[2], m["chebyshev_size"], 1.0, md["coeffs"],
                                 md["linear_coeffs"], md["type_bias"], m["alpha_moments_count"], tb["alpha_index_basic"],
                                 tb["alpha_index_times"], tb["alpha_moment_mapping"], m["nmus"], d["binum"], d["bilist"],
                                 d["bnumneigh"], d["bfirstneigh"], d["brcs"], d["btypes"], tb["type_map"], 0, m["rmax"],
                                 m["rmin"], md["q_scaler"], 0.0, 0.0, None, None, validate=False)
    L = _lib.lib()
    elapsed, kernels = timed(step, args.steps, args.warmup, L)
    _lib.check_status(torch.cuda.current_stream(dev).cuda_stream)
    config = {"workload": args.workload, "natoms": natoms, "structures": B, "natoms_pad": P,
              "model": "linear MTP level 16 K=%d" % m["chebyshev_size"], "species": int(m["type_map"].size),
              "per_step": "normal equations of the linear parameters: components of %d scalar moments + Gram products"
                          % int(m["alpha_moment_mapping"].size)}
    return natoms, elapsed, kernels, None, config, "f64", {}


def cpu_baseline_mtp(cfg):
    import oracle
    from ai2pot_amd import synth
    m, nb, _ = mtp_setup(cfg)
    use_ref = oracle.ref_available("mtpr")
    natoms = int(nb["binum"].sum())
    t0 = time.time()
    if cfg == 4:
        if not use_ref:
            raise RuntimeError("the restatement's forward-mode gradient is too slow to serve as a baseline")
        B, P = nb["bilist"].shape
        lab = dict(energy=synth.rng_normal(4005, B * P, -4.0, 0.2).reshape(B, P).sum(1),
                   force=synth.rng_normal(4006, B * P * 3, 0.0, 1.0).reshape(B, P, 3),
                   virial=synth.rng_normal(4007, B * 9, 0.0, 0.5).reshape(B, 9))
        oracle.ref_mtp_loss_step(m, nb, (1.0, 1.0, 1.0), lab)
        what = "loss forward + backward (the reference's backward recomputes E/F/V once more; not included)"
    else:
        (oracle.ref_mtp_efv if use_ref else oracle.mtp_efv)(m, nb)
        what = "E/F/V"
    dt = time.time() - t0
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return dict(value=natoms / dt, unit="atom-steps/s", cores=threads, kind="reference" if use_ref else "port",
                sample="the full workload (%d atoms), %s, OpenMP %d threads, one run" % (natoms, what, threads))


def run_copy_probe(args):
    """Plain device copy of a known size (1 GiB read, 1 GiB written per step).  It is the yardstick
    for the rocprofv3 FETCH_SIZE / WRITE_SIZE counters the roofline `traffic` figures are scaled by."""
    import torch
    n = 1 << 28
    x = torch.full((n,), 1.0, dtype=torch.float32, device="cuda:0")
    y = torch.empty_like(x)
    for _ in range(args.warmup):
        y.copy_(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y.copy_(x)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    print(json.dumps({"metric": "device copy bandwidth (read + write)", "value": 2 * 4 * n / dt / 1e9, "unit": "GB/s",
                      "bytes_read_per_step": 4 * n, "bytes_written_per_step": 4 * n, "ms_per_step": dt * 1e3,
                      "steps": args.steps, "warmup": args.warmup, "n_gpus": 1}))


WORKLOADS = {
    "nep_md_1048576": lambda a: run_nep_md(a, "fcc", 64),         # the headline configuration (configs[4] of the benchmark definition)
    "nep_md_1048576_ops": lambda a: run_nep_md(a, "fcc", 64, via_ops=True),   # the headline step through torch.ops only
    "nep_md_131072": lambda a: run_nep_md(a, "fcc", 32),
    "nep_efv_4096": lambda a: run_nep_md(a, "random", 4096, rebuild=False),   # configs[1]
    "nep_md_4096": lambda a: run_nep_md(a, "random", 4096),      # configs[1] as a molecular-dynamics step: with list rebuild
    "mtp10_efv_216": lambda a: run_mtp(a, 1),                     # configs[0]
    "mtp20_efv_8192": lambda a: run_mtp(a, 3),                    # configs[2]
    "mtp16_train_64x128": lambda a: run_mtp(a, 4),                # configs[3]
    "nep_train_64x128": run_nep_train,                            # NEP counterpart of configs[3] (not one of the benchmark configurations)
    "mtp16_solver_64x128": run_mtp_solver,                        # linear-solver operator on configs[3]'s structures (extra)
    "hbm_copy_probe": None,                                       # counter calibration, not a workload of the path
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="nep_md_1048576", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="the workload's own timed loop only: skip the short runs of the other benchmark configurations and "
                         "the variants of the step (without padded arrays, through torch.ops)")
    ap.add_argument("--graph", action="store_true",
                    help="time replays of the step captured as a HIP graph (workloads without list rebuild)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported "
                 "(the path has no collectives or sharding)" % args.gpus)
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    if args.workload == "hbm_copy_probe":
        return run_copy_probe(args)

    n, elapsed, kernels, roofline, config, dtype, extra = WORKLOADS[args.workload](args)
    ms_per_step = elapsed * 1e3 / args.steps
    out = {
        "metric": "atom-steps/s (E+F+virial) on 1 MI355X", "value": n * args.steps / elapsed,
        "unit": "atom-steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "us_per_atom_step": ms_per_step * 1e3 / n, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": config,
        "roofline": roofline, "kernels": kernels,
    }
    out.update(extra)
    if args.workload == "nep_md_1048576" and not args.no_other_configs and not args.graph:
        # the remaining benchmark configurations, after the headline's timed region (so they cannot
        # perturb it): ms per step and the roofline entry of the kernel that takes the most time
        import copy
        import torch
        others = {}
        for wl in ("mtp10_efv_216", "nep_efv_4096", "mtp20_efv_8192", "mtp16_train_64x128", "nep_train_64x128",
                   "mtp16_solver_64x128"):
            a2 = copy.copy(args)
            a2.workload, a2.steps, a2.warmup = wl, (5 if "solver" in wl else 50), (1 if "solver" in wl else 5)
            try:
                n2, el2, k2, roof2, _, dt2, _ = WORKLOADS[wl](a2)
                others[wl] = dict(natoms=n2, ms_per_step=el2 * 1e3 / a2.steps, value=n2 * a2.steps / el2,
                                  unit="atom-steps/s", dtype=dt2, steps=a2.steps,
                                  roofline=None if roof2 is None else
                                  {k: roof2.get(k) for k in ("kernel", "bound", "achieved", "peak", "unit", "frac",
                                                             "avg_ms", "traffic", "executed", "executed_frac")})
            except Exception as ex:
                others[wl] = {"error": repr(ex)}
            torch.cuda.synchronize()
        out["other_configs"] = others
    if not args.no_cpu_baseline:
        try:
            if args.workload in ("nep_train_64x128", "mtp16_solver_64x128"):
                out["cpu_baseline"] = {"note": "no CPU baseline leg for this extra workload"}
            elif args.workload.startswith("nep"):
                out["cpu_baseline"] = cpu_baseline_nep()
            else:
                out["cpu_baseline"] = cpu_baseline_mtp({"mtp10_efv_216": 1, "mtp20_efv_8192": 3,
                                                        "mtp16_train_64x128": 4}[args.workload])
        except Exception as ex:       # the baseline is a report, never a reason to lose the GPU line
            out["cpu_baseline"] = {"error": repr(ex)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
