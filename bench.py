"""Benchmark of the fused message-passing convolution, forward + VJP, float32, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg3|cfg2|cfg4]

A step is one pass of the hot path over one batch of synthetic input: the
operator `convolution` (graph preparation + forward kernel) followed by its VJP
through autograd (`convolution_bwd`: cotangents of node features, harmonics and
radial weights)
on the MACE-scale layer: 32 000 atoms, ~30 neighbours (~0.96 M edges), 128
channels, irreps 0e+1o+2e+3o, harmonics up to l = 3, all paths up to l_out = 3,
receiver-sorted edges, trailing-channels layout.  Inputs are resident in HBM
before the timed region.  One JSON line is printed:

  value      edges/s of forward + VJP (whole job, wall clock over K steps)
  roofline   dominant kernel (the backward): algorithmic bytes of one launch /
             its average duration from HIP events on the launch stream, against
             the 8 TB/s HBM peak; forward and combined figures ride along
  cpu_baseline  the C restatement of the reference's CPU loops (OpenMP) timed
             on a bounded sample of the same workload on the host cores
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

#: HBM bytes per launch come from `profiles/traffic.json`: two `rocprofv3 --pmc` runs of this
#: script (FETCH_SIZE and WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads
#: for a 1 GiB device copy (FETCH_SIZE counts half of the bytes read, factor 2.0; WRITE_SIZE all of
#: the bytes written, factor 1.0), written by `python bench.py --write-traffic ...` together with a
#: hash of the kernel sources.  A figure is only quoted while the sources it was
#: measured on are the ones in the tree.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
#: (the sources of the convolution's unrolled kernels: the workloads of the file are convolutions)
KERNEL_SOURCES = ("e3j_amd/csrc/unrolled.h", "e3j_amd/csrc/common.h", "e3j_amd/codegen/gen_conv.py")


def kernel_source_hash() -> str:
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as fh:
            h.update(rel.encode() + b"\0" + fh.read())
    return h.hexdigest()[:16]


def measured_traffic(key: str) -> dict:
    """`{"forward": bytes, "backward": bytes}` for a workload key, {} when there is no measurement of
    the kernels as they are now."""
    try:
        with open(TRAFFIC_FILE) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return {}
    if table.get("kernel_source_hash") != kernel_source_hash():
        return {}
    return table.get("workloads", {}).get(key, {})


def write_traffic(paths, out_path: str, key: str, kernels: dict) -> int:
    """Summarise rocprofv3 counter CSVs (FETCH_SIZE / WRITE_SIZE runs of one bench command) into
    `profiles/traffic.json` under `key`.  `kernels`: pass name -> substring of the kernel name."""
    import csv
    sums = {}
    for path in paths:
        with open(path) as fh:
            for row in csv.DictReader(fh):
                name, counter = row["Kernel_Name"], row["Counter_Name"]
                which = next((k for k, sub in kernels.items() if sub in name), None)
                if which is not None and counter in ("FETCH_SIZE", "WRITE_SIZE"):
                    sums.setdefault((which, counter), []).append(float(row["Counter_Value"]))
    # FETCH_SIZE counts half of the bytes read and WRITE_SIZE all of the bytes written: what the two
    # counters read for a 1 GiB device copy on this GPU (524 300 and 1 048 576 KiB)
    fetch_scale, write_scale = 2.0, 1.0
    entry = {"fetch_scale": round(fetch_scale, 3), "write_scale": round(write_scale, 3)}
    for which in kernels:
        f = sums.get((which, "FETCH_SIZE"), [])
        w = sums.get((which, "WRITE_SIZE"), [])
        if f and w:
            fetch, write = sum(f) / len(f), sum(w) / len(w)
            entry[which] = (fetch_scale * fetch + write_scale * write) * 1024.0
            entry[which + "_counters_KiB"] = {"FETCH_SIZE": fetch, "WRITE_SIZE": write}
    try:
        with open(out_path) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        table = {}
    if table.get("kernel_source_hash") != kernel_source_hash():
        table = {"kernel_source_hash": kernel_source_hash(), "workloads": {}}
    table["workloads"][key] = entry
    with open(out_path, "w") as fh:
        json.dump(table, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print(json.dumps({key: entry}))
    return 0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="cfg3", choices=["cfg2", "cfg3", "cfg4", "cfg5"],
                    help="cfg3: the headline workload; cfg2 / cfg4: the other single-convolution "
                         "configurations; cfg5: a secondary figure, energy and forces of the two-layer model")
    ap.add_argument("--layout", default="trailing", choices=["trailing", "leading"],
                    help="memory layout of the node and edge arrays (channels last or first)")
    ap.add_argument("--channels", type=int, default=None,
                    help="channel count of cfg3 (default 128; kernels are built for 32, 64, 128, 256)")
    ap.add_argument("--scale", type=float, default=1.0, help="fraction of the configuration's atoms")
    ap.add_argument("--dtype", default="f32", choices=["f32", "f64", "f16"],
                    help="f64 / f16: the same workload with float64 / float16 operands (secondary figures: the "
                         "float64 and float16 unrolled kernels of the trailing layout)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-layouts", action="store_true",
                    help="skip the leading-channels sub-record of the default run")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--table-driven", action="store_true",
                    help="time the table-driven kernels (signature -1) through the C ABI instead of the unrolled "
                         "ones (implies --kernel-only); E3J_AMD_TABLE_PLANS=0 selects their form without a plan")
    ap.add_argument("--kernel-only", action="store_true",
                    help="time the C-ABI launches only (no operator-level step)")
    ap.add_argument("--deterministic", action="store_true",
                    help="time the atomic-free (bit-reproducible) backward instead of the default one")
    ap.add_argument("--inner", type=int, default=64, help="--op radial_linear: hidden size of the radial network")
    ap.add_argument("--op", default="convolution", choices=["convolution", "tensor_product", "radial_linear"],
                    help="convolution: the headline benchmark; tensor_product: a secondary figure, the "
                         "row-wise product on the same table (0e+1o+2e+3o squared, l <= 3, 128 channels)")
    ap.add_argument("--mode", default="MAP", choices=["MAP", "OUTER", "INNER"],
                    help="--op tensor_product: channel mode (OUTER: y without channel axis)")
    ap.add_argument("--rows", type=int, default=1 << 18, help="--op tensor_product: number of rows")
    ap.add_argument("--write-traffic", nargs="+", metavar="CSV",
                    help="no GPU work: summarise rocprofv3 counter CSVs (FETCH_SIZE and WRITE_SIZE runs of this "
                         "script) into profiles/traffic.json for --config/--layout/--scale")
    return ap.parse_args()


def build_workload(name: str, scale: float, device, channels=None):
    from e3j_amd import workloads as W
    if name == "cfg2":
        return W.config2(scale, device=device)
    if name == "cfg4":
        return W.config4(scale, device=device)
    return W.config3(scale, device=device, **({"channels": channels} if channels else {}))


class AbiCalls:
    """Direct launches through the C ABI with a prebuilt receiver CSR (kernel timing)."""

    def __init__(self, w, table_driven=False, paired=False):
        import numpy as np
        import torch
        from e3j_amd import _lib
        from e3j_amd.graph import csr_row_ptr, locality_order, sort_edges
        from e3j_amd.options import config
        from e3j_amd.ops import _Table
        self.torch, self.lib, self._lib = torch, _lib.load(), _lib
        self.w = w
        module = w.module
        packed = module._packed_coef("float32")
        self.table = _Table.get(packed, np.float32)
        d = 2 if w.leading else 1
        dims = (w.x.shape[d], w.y.shape[1], module.params.num_out, w.s.shape[d])
        sig, scale, _ = self.table.signature(tuple(int(d) for d in dims), w.channels, module.layout)
        if table_driven:   # the kernels that read the table at run time, as for a table without a signature
            sig, scale = -1, 1.0
        self.signature = sig
        self.params = _lib.ConvParams(
            num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=self.table.num_coef,
            num_x=int(dims[0]), num_y=int(dims[1]), num_out=int(dims[2]), num_scalars=int(dims[3]),
            channels=w.channels, layout=module.layout.value, val_dtype=_lib.F32,
            coef_idx_bytes=self.table.idx_bytes, signature=sig, coef_scale=scale, debug=0)
        self.coef = self.table.device(w.x.device)
        if table_driven:   # the plan of the table built once, as the operators do on a table's first call
            nbytes = int(self.lib.e3j_amd_table_plan_bytes(ctypes.byref(self.params)))
            if nbytes:
                self.plan = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device=w.x.device)
                self.params.table_plan = self.plan.data_ptr()
                status = (ctypes.c_int32 * 4)()
                _lib.check(self.lib.e3j_amd_table_plan_status(ctypes.byref(self.params), self.coef.data_ptr(), 0,
                                                              status, int(torch.cuda.current_stream().cuda_stream)))
                if not status[0]:
                    self.params.table_plan = None
                self.params.table_plan_state = _lib.PLAN_READY if status[0] else _lib.PLAN_NONE
        if module.graph_ordering.value == "NONE":
            self.perm, self.other, self.ptr = sort_edges(w.receiver, w.sender, w.num_nodes)
        else:
            self.perm, self.other = None, w.sender.contiguous()
            self.ptr = csr_row_ptr(w.receiver, w.num_nodes)
        rounds = config().locality_rounds
        self.order = locality_order(self.other, self.ptr, w.num_nodes, rounds) if rounds > 0 else None
        if self.order is not None and (paired or config().pair_rows is True):   # as the operators do
            from e3j_amd.graph import pair_rows
            self.order = pair_rows(self.other, self.ptr, w.num_nodes, self.order)
        self.params.row_order = self.order.data_ptr() if self.order is not None else None
        self.out = torch.empty_like(w.dm)
        self.dx, self.dy, self.ds = torch.empty_like(w.x), torch.empty_like(w.y), torch.empty_like(w.s)
        # the default backward of the operators: tiles of receivers when the signature has such a kernel
        self.schedule = None
        from e3j_amd.ops import _tile_rows
        tile_rows = _tile_rows(sig) if module.layout.value == _lib.LAYOUT_TRAILING else 0
        self.tile_rows = tile_rows
        if tile_rows >= 1:
            from e3j_amd.graph import TileSchedule
            self.schedule = TileSchedule(self.other, self.ptr, self.perm, self.order, w.num_nodes, tile_rows)

    def _stream(self):
        return int(self.torch.cuda.current_stream().cuda_stream)

    def forward(self):
        w = self.w
        self._lib.check(self.lib.e3j_amd_convolution_fwd(
            ctypes.byref(self.params), self.coef.data_ptr(), w.x.data_ptr(), w.y.data_ptr(),
            w.s.data_ptr(), self.other.data_ptr(), self.ptr.data_ptr(),
            self.perm.data_ptr() if self.perm is not None else None, self.out.data_ptr(),
            self._stream()))

    def backward_ordered(self):
        w = self.w
        if not hasattr(self, "workspace"):
            nbytes = int(self.lib.e3j_amd_convolution_bwd_ordered_workspace_bytes(ctypes.byref(self.params)))
            self.workspace = self.torch.empty(nbytes, dtype=self.torch.uint8, device=w.x.device)
        self._lib.check(self.lib.e3j_amd_convolution_bwd_ordered(
            ctypes.byref(self.params), self.coef.data_ptr(), w.x.data_ptr(), w.y.data_ptr(),
            w.s.data_ptr(), w.dm.data_ptr(), self.other.data_ptr(), self.ptr.data_ptr(),
            self.perm.data_ptr() if self.perm is not None else None,
            self.dx.data_ptr(), self.dy.data_ptr(), self.ds.data_ptr(), self.workspace.data_ptr(),
            self._stream()))

    def backward(self):
        """The backward the operators run by default."""
        if self.schedule is None:
            return self.backward_receiver()
        w = self.w
        self._lib.check(self.lib.e3j_amd_convolution_bwd_tiled(
            ctypes.byref(self.params), w.x.data_ptr(), w.y.data_ptr(), w.s.data_ptr(), w.dm.data_ptr(),
            self.other.data_ptr(), self.ptr.data_ptr(), self.perm.data_ptr() if self.perm is not None else None,
            ctypes.byref(self.schedule.struct), self.dx.data_ptr(), self.dy.data_ptr(), self.ds.data_ptr(),
            self._stream()))

    def backward_receiver(self):
        """One wave per (receiver, slice, part), one set of dx atomics per edge."""
        w = self.w
        self._lib.check(self.lib.e3j_amd_convolution_bwd_receiver(
            ctypes.byref(self.params), self.coef.data_ptr(), w.x.data_ptr(), w.y.data_ptr(),
            w.s.data_ptr(), w.dm.data_ptr(), self.other.data_ptr(), self.ptr.data_ptr(),
            self.perm.data_ptr() if self.perm is not None else None,
            self.dx.data_ptr(), self.dy.data_ptr(), self.ds.data_ptr(), self._stream()))


def time_events(torch, fn, steps: int, warmup: int, stats: dict | None = None) -> float:
    """Average milliseconds of `fn` from HIP events recorded on the launch stream (`stats`, if given,
    also receives the median and the minimum)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for a, b in zip(starts, stops):
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) for a, b in zip(starts, stops))
    if stats is not None:
        stats.update(ms_median=times[len(times) // 2], ms_min=times[0])
    return sum(times) / steps


def cpu_baseline(w, seconds: float) -> dict:
    """Time the C restatement of the reference loops on a bounded head of the workload."""
    import numpy as np
    from oracle import c_oracle
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    os.environ["OMP_NUM_THREADS"] = str(cores)
    idx, val, mix = w.table()
    num_out = w.module.params.num_out

    def run(num_receivers):
        h = w.head(num_receivers)
        a = h.numpy()
        x, dm = a["x"], a["dm"]
        t0 = time.perf_counter()
        c_oracle.convolution(idx, val, mix, x, a["y"], a["s"], a["sender"], a["receiver"], num_out)
        c_oracle.convolution_vjp(idx, val, mix, x, a["y"], a["s"], a["sender"], a["receiver"], dm)
        return h.num_edges, time.perf_counter() - t0

    # grow the sample until it takes about `seconds` (the first calls pay thread start-up)
    want_nodes = min(w.num_nodes, 256)
    edges, t = run(want_nodes)
    for _ in range(4):
        if t >= 0.6 * seconds or want_nodes >= w.num_nodes:
            break
        want_nodes = int(min(w.num_nodes, max(2 * want_nodes, want_nodes * seconds / max(t, 1e-3))))
        edges, t = run(want_nodes)
    return {"value": edges / t, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": f"forward + VJP on the edges of the first {want_nodes} receivers "
                      f"({edges} edges) of the same workload, {t:.1f} s"}


#: the same for `--op tensor_product` (MAP, trailing layout, 262 144 rows, 128 channels)
MEASURED_TP_TRAFFIC_BYTES = {
    ("MAP", "trailing", 1 << 18, 128): {"forward": 2.0 * 2.097e6 * 1024 + 1.299e7 * 1024,
                                        "backward": 2.0 * 8.585e6 * 1024 + 4.194e6 * 1024},
}


def bench_other_dtype(args, torch, device) -> int:
    """Secondary figure: forward + VJP with float64 or float16 operands through the operators (graph
    preparation in every step), the unrolled kernels of that dtype timed on their own through the C
    ABI, and the table-driven kernels, which served these dtypes before, on an eighth of the workload."""
    import numpy as np
    import e3j_amd
    from e3j_amd import _lib
    from e3j_amd.graph import csr_row_ptr, locality_order
    from e3j_amd.ops import _Table, clear_graph_cache
    lib = _lib.load()
    f64 = args.dtype == "f64"
    tdtype, ndtype, code, name = ((torch.float64, np.float64, _lib.F64, "float64") if f64
                                  else (torch.float16, np.float16, _lib.F16, "float16"))
    shrink = 1.0 if f64 else 0.25   # (sums of thirty messages stay inside the half range)

    def calls(w):
        module = w.module
        table = _Table.get(module._packed_coef(name), ndtype)
        dims = (int(w.x.shape[1]), int(w.y.shape[1]), module.params.num_out, int(w.s.shape[1]))
        sig, classes, flip = table.signature(dims, w.channels, module.layout)
        x, y, s, dm = ((t * shrink).to(tdtype) for t in (w.x, w.y, w.s, w.dm))
        ptr = csr_row_ptr(w.receiver, w.num_nodes)
        order = locality_order(w.sender, ptr, w.num_nodes, 2)
        out, dx, dy, ds = (torch.empty_like(t) for t in (dm, x, y, s))
        coef = table.device(device)
        keep_t = []
        keep = (x, y, s, dm, ptr, order, out, dx, dy, ds, coef, classes, keep_t)

        def params(signature):
            p = _lib.ConvParams(num_nodes=w.num_nodes, num_edges=w.num_edges, num_coef=table.num_coef,
                                num_x=dims[0], num_y=dims[1], num_out=dims[2], num_scalars=dims[3],
                                channels=w.channels, layout=module.layout.value, val_dtype=code,
                                coef_idx_bytes=table.idx_bytes, signature=signature,
                                coef_scale=classes if isinstance(classes, float) and signature >= 0 else 1.0,
                                debug=0, y_flip=flip if signature >= 0 else 0)
            p.row_order = order.data_ptr()
            if signature >= 0 and f64:
                p.coef_classes = ctypes.cast(classes, ctypes.c_void_p).value
            return p

        def pair(p):
            stream = lambda: int(torch.cuda.current_stream().cuda_stream)  # noqa: E731
            fwd = lambda: _lib.check(lib.e3j_amd_convolution_fwd(  # noqa: E731
                ctypes.byref(p), coef.data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(), w.sender.data_ptr(),
                ptr.data_ptr(), None, out.data_ptr(), stream()))
            bwd = lambda: _lib.check(lib.e3j_amd_convolution_bwd_receiver(  # noqa: E731
                ctypes.byref(p), coef.data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(),
                w.sender.data_ptr(), ptr.data_ptr(), None, dx.data_ptr(), dy.data_ptr(), ds.data_ptr(), stream()))
            if p.signature < 0 and not f64:
                # the table-driven kernels add dx with float atomics, which have no half form: their
                # float16 backward runs on the sender-grouped adjacency, whose rows own their dx
                from e3j_amd.graph import sort_edges
                tperm, tother, tptr = sort_edges(w.sender, w.receiver, w.num_nodes)
                keep_t.extend((tperm, tother, tptr))
                bwd = lambda: _lib.check(lib.e3j_amd_convolution_bwd_sender(  # noqa: E731
                    ctypes.byref(p), coef.data_ptr(), x.data_ptr(), y.data_ptr(), s.data_ptr(), dm.data_ptr(),
                    tother.data_ptr(), tptr.data_ptr(), tperm.data_ptr(), dx.data_ptr(), dy.data_ptr(), ds.data_ptr(),
                    stream()))
            return fwd, bwd
        return sig, params, pair, keep

    w = build_workload(args.config, args.scale, device, args.channels)
    if w.module.graph_ordering.value == "NONE" or args.layout != "trailing":
        print("bench.py --dtype f64 / f16 times receiver-ordered workloads in the trailing layout", file=sys.stderr)
        return 2
    module = w.module
    coef = module._packed_coef(name)
    sig, params, pair, keep = calls(w)
    if sig < 0:
        print(f"bench.py --dtype {args.dtype}: no {name} unrolled kernel for this table", file=sys.stderr)
        return 2
    xg, yg, sg = (t.requires_grad_(True) for t in keep[:3])
    dm = keep[3]

    def step():
        clear_graph_cache()
        out = e3j_amd.convolution(coef, xg, yg, sg, w.sender, w.receiver, module.params, module.graph_ordering,
                                  layout=module.layout)
        return out, torch.autograd.grad(out, (xg, yg, sg), dm)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    fwd, bwd = pair(params(sig))
    fwd_ms, bwd_ms = time_events(torch, fwd, args.steps, 2), time_events(torch, bwd, args.steps, 2)
    b32 = w.algorithmic_bytes()
    index_bytes = {"fwd": 4 * (w.num_edges + w.num_nodes + 1), "bwd": 4 * (2 * w.num_edges + w.num_nodes + 1)}
    width = 2.0 if f64 else 0.5
    b64 = {k: int(width * (b32[k] - index_bytes[k])) + index_bytes[k] for k in ("fwd", "bwd")}   # values resized, indices as they are
    frac = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS  # noqa: E731
    result = {
        "metric": f"edges/sec fused Convolution fwd+VJP {'fp64' if f64 else 'fp16'}", "value": w.num_edges / (ms_per_step * 1e-3),
        "unit": "edges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"{args.config} x {args.scale}: {w.num_nodes} atoms, {w.num_edges} edges, K={w.channels}, "
                               f"{name} operands, receiver-ordered edges, trailing-channels layout, forward + VJP",
                   "signature": sig},
        "roofline": {"bound": "hbm", "kernel": f"convolution backward, {name} (unrolled_bwd_{args.dtype}_kernel + dx, dy zero fills)",
                     "achieved": b64["bwd"] / (bwd_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": frac(b64["bwd"], bwd_ms), "traffic": None, "algorithmic_bytes": b64["bwd"], "ms": bwd_ms,
                     "forward": {"ms": fwd_ms, "algorithmic_bytes": b64["fwd"], "frac": frac(b64["fwd"], fwd_ms)}},
        "cpu_baseline": None,
    }
    del keep, xg, yg, sg, dm, fwd, bwd
    small = build_workload(args.config, args.scale * 0.125, device, args.channels)
    ssig, sparams, spair, skeep = calls(small)
    record = {"workload": f"{args.config} x {args.scale * 0.125}: {small.num_edges} edges, K={small.channels}", "unit": "ms"}
    for name, signature in (("unrolled", ssig), ("table_driven", -1)):
        f, b = spair(sparams(signature))
        record[name] = {"forward": time_events(torch, f, 5, 1), "backward": time_events(torch, b, 5, 1)}
    result["table_driven"] = record
    print(json.dumps(result))
    return 0


def bench_energy(args, torch, device) -> int:
    """Secondary figure: energy and forces of the two-layer model (positions -> harmonics and
    radial weights -> two convolutions with channel mixing -> scalar energy; forces by autograd
    through the kernels' VJPs).  The roofline entry is the backward kernel of one of its layers."""
    from e3j_amd import workloads as W
    wl = W.config5(args.scale)
    d = wl.to(device, torch.float32)
    model = wl.model

    def step():
        return model.energy_and_forces(d.positions, d.node_features, d.sender, d.receiver, d.shift)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # one layer's convolution on the model's own operands, through the C ABI
    with torch.no_grad():
        y, basis = model.edge_inputs(d.positions, d.sender, d.receiver, d.shift)
        w1, w2 = (torch.as_tensor(a, dtype=torch.float32, device=device) for a in model.mlp[0])
        s = (torch.nn.functional.silu(basis @ w1) @ w2).reshape(-1, model.num_paths, model.channels).contiguous()
    layer = model.layers[0]
    dm = torch.randn((d.node_features.shape[0], layer.target.dim, model.channels), device=device,
                     generator=torch.Generator(device=device).manual_seed(0))
    w = W.Workload("cfg5 layer", layer, d.node_features.contiguous(), y.contiguous(), s, dm, d.sender, d.receiver,
                   wl.positions.numpy(), 0.0)
    abi = AbiCalls(w)
    fwd_ms = time_events(torch, abi.forward, args.steps, 2)
    bwd_ms = time_events(torch, abi.backward, args.steps, 2)
    bytes_ = w.algorithmic_bytes()

    def gbs(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9

    result = {
        "metric": "edges/sec energy + forces, two fused Convolution layers, fp32",
        "value": wl.num_edges / (ms_per_step * 1e-3), "unit": "edges/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"cfg5: {d.positions.shape[0]} atoms in a periodic box, {wl.num_edges} edges, two "
                               f"convolutions ({model.channels} channels, 0e+1o+2e+3o, l <= 3) with channel mixing, "
                               "radial weights from an MLP over 8 Bessel functions, scalar energy, forces by "
                               "autograd with respect to the positions",
                   "scale": args.scale, "signature": abi.signature},
        "roofline": {"bound": "hbm", "kernel": "convolution backward of one layer (unrolled_bwd_kernel + dx zero fill)",
                     "achieved": gbs(bytes_["bwd"], bwd_ms), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs(bytes_["bwd"], bwd_ms) / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes": bytes_["bwd"], "ms": bwd_ms,
                     "forward": {"achieved": gbs(bytes_["fwd"], fwd_ms), "frac": gbs(bytes_["fwd"], fwd_ms) / HBM_PEAK_GBS,
                                 "traffic": None, "algorithmic_bytes": bytes_["fwd"], "ms": fwd_ms},
                     "convolution_kernels_ms_per_step": 2 * (fwd_ms + bwd_ms)},
        "cpu_baseline": None,
    }
    print(json.dumps(result))
    return 0


def bench_radial_linear(args, torch, device) -> int:
    """Secondary figure: the last layer of the radial network, s = h W on the matrix cores, at the
    edge count and paths * channels of the headline workload; beside it the library product."""
    from e3j_amd.radial import radial_linear
    edges, n, inner = int(959970 * args.scale), 23 * (args.channels or 128), args.inner
    g = torch.Generator(device=device).manual_seed(0)
    h = torch.randn(edges, inner, device=device, generator=g)
    w = torch.randn(inner, n, device=device, generator=g)
    out = torch.empty(edges, n, device=device)
    ms = time_events(torch, lambda: radial_linear(h, w), args.steps, args.warmup)
    lib_ms = time_events(torch, lambda: torch.matmul(h, w, out=out), args.steps, args.warmup)
    nbytes = 4 * (edges * n + edges * inner + inner * n)
    flops = 2.0 * edges * inner * n
    split = inner >= 64   # three-way bfloat16 split: six matrix-core products per float32 product
    result = {
        "metric": "edges/sec radial network last layer (s = h W) fp32", "value": edges / (ms * 1e-3),
        "unit": "edges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"s ({edges}, {n}) = h ({edges}, {inner}) W ({inner}, {n}), float32"
                               + (", operands split three ways on the bfloat16 matrix cores" if split else
                                  ", float32 matrix-core products")},
        "roofline": {"bound": "hbm", "kernel": "radial_linear_fwd" + ("_split" if split else "") + "_kernel",
                     "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes": nbytes,
                     "ms": ms,
                     "matrix_cores": {"flop": flops, "products_per_float32_product": 6 if split else 1,
                                      "achieved_tflops": flops * (6 if split else 1) / (ms * 1e-3) / 1e12,
                                      "peak_tflops": 2500.0 if split else 157.3},
                     "library_product_ms": lib_ms},
        "cpu_baseline": None,
    }
    print(json.dumps(result))
    return 0


def bench_tensor_product(args, torch, device) -> int:
    """Secondary figure: the row-wise tensor product (forward + VJP) on the benchmark's table."""
    import numpy as np
    import e3j_amd
    from e3j_amd import TensorProduct
    from e3j_amd.tp_ops import TensorProductParams, _make_meta, _params, _raw_backward, _raw_forward
    layout = "LEADING_CHANNELS" if args.layout == "leading" else "TRAILING_CHANNELS"
    trailing = layout == "TRAILING_CHANNELS"
    K, R = args.channels or 128, args.rows
    tp = TensorProduct(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", layout=layout, mode=args.mode)
    Z, X, Y = tp.shape
    name = {"f32": "float32", "f64": "float64", "f16": "float16"}[args.dtype]
    tdtype = getattr(torch, name)
    coef = tp.packed_coef(name)
    params = TensorProductParams(num_out=Z, mode=args.mode, layout=layout)
    g = torch.Generator(device=device).manual_seed(0)
    x = torch.randn((R, X, K) if trailing else (R, K, X), device=device, generator=g).to(tdtype)
    has_cy = args.mode != "OUTER"
    y = torch.randn(((R, Y, K) if trailing else (R, K, Y)) if has_cy else (R, Y), device=device, generator=g).to(tdtype)
    meta = _make_meta(coef, x, y, params)
    z = _raw_forward(meta, x, y)
    dz = torch.randn(tuple(z.shape), device=device, generator=g).to(tdtype)
    signature = _params(meta, x, y, backward=False).signature
    xg, yg = x.detach().requires_grad_(True), y.detach().requires_grad_(True)

    def step():
        out = e3j_amd.tensor_product(coef, xg, yg, params)
        return torch.autograd.grad(out, (xg, yg), dz)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    fwd_ms = time_events(torch, lambda: _raw_forward(meta, x, y), args.steps, 2)
    bwd_ms = time_events(torch, lambda: _raw_backward(meta, x, y, dz), args.steps, 2)
    width = x.element_size()
    fwd_bytes = width * (x.numel() + y.numel() + z.numel())
    bwd_bytes = width * (2 * x.numel() + 2 * y.numel() + z.numel())

    def gbs(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9

    measured = MEASURED_TP_TRAFFIC_BYTES.get((args.mode, args.layout, R, K), {}) if args.dtype == "f32" else {}
    result = {
        "metric": "rows/sec fused TensorProduct fwd+VJP " + args.dtype.replace("f", "fp") + "; achieved HBM GB/s vs peak",
        "value": R / (ms_per_step * 1e-3), "unit": "rows/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"row-wise tensor product 0e+1o+2e+3o (x) 0e+1o+2e+3o -> l <= 3 ({len(tp.values)} "
                               f"coefficients, {Z} output coordinates), {R} rows, {K} channels, mode {args.mode}, "
                               f"{args.layout}-channels layout, forward + VJP (dx, dy)",
                   "signature": signature,
                   "signature_name": (_lib_name(signature) if signature >= 0 else "table-driven kernel")},
        "roofline": {"bound": "hbm", "kernel": "tensor product backward (dz read once for dx and dy)",
                     "achieved": gbs(bwd_bytes, bwd_ms), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs(bwd_bytes, bwd_ms) / HBM_PEAK_GBS, "traffic": measured.get("backward"),
                     "algorithmic_bytes": bwd_bytes, "ms": bwd_ms,
                     "forward": {"achieved": gbs(fwd_bytes, fwd_ms), "frac": gbs(fwd_bytes, fwd_ms) / HBM_PEAK_GBS,
                                 "traffic": measured.get("forward"),
                                 "algorithmic_bytes": fwd_bytes, "ms": fwd_ms},
                     "forward_plus_backward": {"achieved": gbs(fwd_bytes + bwd_bytes, fwd_ms + bwd_ms),
                                               "frac": gbs(fwd_bytes + bwd_bytes, fwd_ms + bwd_ms) / HBM_PEAK_GBS,
                                               "algorithmic_bytes": fwd_bytes + bwd_bytes, "ms": fwd_ms + bwd_ms}},
    }
    if not args.no_cpu_baseline:
        from oracle import tp_oracle
        idx, val = np.asarray(tp.indices, dtype=np.int64), np.asarray(tp.values, dtype=np.float32)
        rows = 2048
        xs, ys, dzs = (t[:rows].float().cpu().numpy() for t in (x, y, dz))
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < args.cpu_seconds:
            tp_oracle.tensor_product_unfused(idx, val, xs, ys, Z, args.mode, layout)
            tp_oracle.tensor_product_vjp(idx, val, xs, ys, dzs, args.mode, layout)
            reps += 1
        elapsed = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": rows * reps / elapsed, "unit": "rows/s", "cores": 1, "kind": "port",
                                  "sample": f"forward + VJP of the numpy restatement on the first {rows} rows, "
                                            f"{reps} repetitions, {elapsed:.1f} s"}
    print(json.dumps(result))
    return 0


def _lib_name(signature: int) -> str:
    from e3j_amd import _lib
    return _lib.load().e3j_amd_tp_signature_name(signature).decode()


def traffic_key(args, tiled=None) -> str:
    """Key of a measurement: workload, layout and which backward kernel ran."""
    if tiled is None:  # what the library does by default for the trailing layout
        tiled = args.layout == "trailing" and not args.deterministic
    return f"{args.config}/{args.scale}/{args.layout}/k{args.channels or 'default'}" + ("/tiled" if tiled else "")


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        return 2
    if args.write_traffic:
        key = traffic_key(args)
        names = ({"forward": "unrolled_fwd_leading", "backward": "unrolled_bwd_leading"} if args.layout == "leading"
                 else {"forward": "unrolled_fwd_kernel",
                       "backward": "unrolled_bwd_tile_kernel" if key.endswith("/tiled") else "unrolled_bwd_kernel"})
        return write_traffic(args.write_traffic, TRAFFIC_FILE, key, names)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no GPU is visible", file=sys.stderr)
        return 2
    import e3j_amd
    from e3j_amd import _lib
    _lib.load()  # fail loudly when the HIP library is missing
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.op == "tensor_product":
        return bench_tensor_product(args, torch, device)
    if args.op == "radial_linear":
        return bench_radial_linear(args, torch, device)
    if args.config == "cfg5":
        return bench_energy(args, torch, device)
    if args.dtype != "f32":
        return bench_other_dtype(args, torch, device)

    w = build_workload(args.config, args.scale, device, args.channels)
    w = w.with_layout("LEADING_CHANNELS" if args.layout == "leading" else "TRAILING_CHANNELS")
    module = w.module
    coef = module._packed_coef("float32")
    bytes_ = w.algorithmic_bytes(sorted_edges=module.graph_ordering.value != "NONE")

    xg, yg, sg = (t.detach().requires_grad_(True) for t in (w.x, w.y, w.s))

    from e3j_amd.ops import clear_graph_cache

    def step():
        # forward, then the VJP of (x, y, s) for the cotangent dm, as autograd runs them; the
        # adjacency is prepared anew in every step (no reuse between steps)
        clear_graph_cache()
        out = e3j_amd.convolution(coef, xg, yg, sg, w.sender, w.receiver, module.params,
                                  module.graph_ordering, layout=module.layout)
        grads = torch.autograd.grad(out, (xg, yg, sg), w.dm)
        return out, grads

    if args.table_driven:
        args.kernel_only = True   # the operators resolve the table to its unrolled kernels
    abi = AbiCalls(w, table_driven=args.table_driven)
    if args.deterministic:
        e3j_amd.config(deterministic=True)
        abi.backward = abi.backward_ordered
    if args.kernel_only:
        def step():  # noqa: F811
            abi.forward()
            abi.backward()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    fwd_stats, bwd_stats = {}, {}
    fwd_ms = time_events(torch, abi.forward, args.steps, 2, fwd_stats)
    bwd_ms = time_events(torch, abi.backward, args.steps, 2, bwd_stats)

    # graph preparation of one step (row pointers, row order; the reference pays its bincount, cumsum
    # and argsort inside the operator too): part of `ms_per_step`, reported on its own as well
    from e3j_amd.ops import prepare_graph
    prep_stats = {}
    def prepare():
        # as inside an operator call: without the row pairing that handles built once get by default
        g = prepare_graph(w.sender, w.receiver, w.num_nodes, module.graph_ordering, pair_rows=False)
        if abi.schedule is not None:
            g.schedule(abi.tile_rows)
    prep_ms = time_events(torch, prepare, args.steps, 2, prep_stats)

    def gbs(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9

    tiled = abi.schedule is not None and not args.deterministic
    measured = {} if args.deterministic else measured_traffic(traffic_key(args, tiled))
    bwd_gbs, fwd_gbs = gbs(bytes_["bwd"], bwd_ms), gbs(bytes_["fwd"], fwd_ms)
    both_gbs = gbs(bytes_["fwd_bwd"], fwd_ms + bwd_ms)
    result = {
        "metric": "edges/sec fused Convolution fwd+VJP fp32; achieved HBM GB/s vs peak",
        "value": w.num_edges / (ms_per_step * 1e-3),
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{args.config}: {w.num_nodes} atoms, {w.num_edges} edges, K={w.channels}, "
                        f"x {module.source[0]}, y {module.source[1]}, out {module.target}, "
                        f"{module.graph_ordering.value.lower()}-ordered edges, {args.layout}-channels layout, "
                        "forward + VJP (dx, dy, ds)",
            "scale": args.scale,
            "atom_numbering": "random",
            "signature": abi.signature,
            "signature_name": (_lib.load().e3j_amd_signature_name(abi.signature).decode()
                               if abi.signature >= 0 else "table-driven kernel"),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": ("convolution backward, table-driven (plan_build_kernel + planned_bwd_kernel + dx zero fill)"
                       if abi.signature < 0 else
                       "convolution backward, atomic-free (position sort + unrolled_bwd_kernel + fixed-order "
                       "dx/dy reductions)" if args.deterministic else
                       "convolution backward over tiles of receivers (unrolled_bwd_tile_kernel + dx zero fill)"
                       if tiled else "convolution backward (unrolled_bwd_kernel + dx zero fill)"),
            "achieved": bwd_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bwd_gbs / HBM_PEAK_GBS,
            "traffic": measured.get("backward"),
            "algorithmic_bytes": bytes_["bwd"], "ms": bwd_ms, **bwd_stats,
            "forward": {"achieved": fwd_gbs, "frac": fwd_gbs / HBM_PEAK_GBS,
                        "traffic": measured.get("forward"),
                        "algorithmic_bytes": bytes_["fwd"], "ms": fwd_ms, **fwd_stats},
            "forward_plus_backward": {"achieved": both_gbs, "frac": both_gbs / HBM_PEAK_GBS,
                                      "algorithmic_bytes": bytes_["fwd_bwd"], "ms": fwd_ms + bwd_ms},
            "graph_preparation": {"ms": prep_ms, **prep_stats,
                                  "what": "index wrap, row pointers, row order, tile schedule of the backward (per step; "
                                          "included in ms_per_step)"},
        },
    }
    if not args.kernel_only and not args.table_driven and not args.deterministic:
        # the same step for a caller that holds the adjacency across calls (the layers of a model, the
        # steps between two neighbour-list rebuilds): prepared once, outside the timed region, with rows
        # that share senders paired (the default of `prepare_graph`); `value` above prepares per step
        handle = prepare_graph(w.sender, w.receiver, w.num_nodes, module.graph_ordering)

        def held_step():
            out = e3j_amd.convolution(coef, xg, yg, sg, w.sender, w.receiver, module.params,
                                      module.graph_ordering, layout=module.layout, graph=handle)
            return torch.autograd.grad(out, (xg, yg, sg), w.dm)

        for _ in range(args.warmup):
            held_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            held_step()
        torch.cuda.synchronize()
        held_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        paired = AbiCalls(w, paired=True)
        pb_stats = {}
        pb = time_events(torch, paired.backward, args.steps, 2, pb_stats)
        result["prepared_graph"] = {
            "what": "forward + VJP through the operators with a prepare_graph handle built once "
                    "(row pairing on): no graph preparation inside the step",
            "ms_per_step": held_ms, "value": w.num_edges / (held_ms * 1e-3), "unit": "edges/s",
            "frac": gbs(bytes_["fwd_bwd"], held_ms) / HBM_PEAK_GBS,
            "backward": {"ms": pb, **pb_stats, "frac": gbs(bytes_["bwd"], pb) / HBM_PEAK_GBS}}
        del handle, paired
    if args.layout == "trailing" and not args.kernel_only and not args.no_layouts and args.config in ("cfg2", "cfg3"):
        # the same workload in the leading-channels layout (the configurations name both), kernels only
        del abi
        wl = w.with_layout("LEADING_CHANNELS")
        lead = AbiCalls(wl)
        ls_f, ls_b = {}, {}
        lf = time_events(torch, lead.forward, args.steps, 2, ls_f)
        lb = time_events(torch, lead.backward, args.steps, 2, ls_b)
        result["layouts"] = {"leading": {
            "forward": {"ms": lf, **ls_f, "frac": gbs(bytes_["fwd"], lf) / HBM_PEAK_GBS},
            "backward": {"ms": lb, **ls_b, "frac": gbs(bytes_["bwd"], lb) / HBM_PEAK_GBS},
            "forward_plus_backward": {"ms": lf + lb, "frac": gbs(bytes_["fwd_bwd"], lf + lb) / HBM_PEAK_GBS}}}
        del lead, wl
        abi = AbiCalls(w)
    if (args.layout == "trailing" and not args.kernel_only and not args.no_layouts and args.config == "cfg3"
            and args.scale == 1.0 and not args.table_driven):
        # the kernels that read the table at run time (a table without built-in kernels on a host
        # without hipcc), at an eighth of the workload, beside the unrolled kernels on the same inputs
        small = build_workload(args.config, 0.125, device, channels=args.channels)
        record = {"workload": f"{args.config} x 0.125: {small.num_nodes} atoms, {small.num_edges} edges, "
                              f"K={small.channels}", "unit": "ms"}
        for name, flag in (("table_driven", True), ("unrolled", False)):
            calls = AbiCalls(small, table_driven=flag)
            record[name] = {"forward": time_events(torch, calls.forward, args.steps, 2),
                            "backward": time_events(torch, calls.backward, args.steps, 2)}
            del calls
        result["table_driven"] = record
        del small
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, args.cpu_seconds)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
