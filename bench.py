"""Benchmark of the scan hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one forward scan plus one fused backward scan over the same
synthetic batch, both through the C ABI with every buffer already resident in
HBM.  The default workload is the headline configuration: fp32, shape
(8, 1536, 65536), inputs drawn as the reference's benchmark draws them
(tests/bench.py:6-11 of the reference: seed 12312323, gates
0.999 + 0.001 U rounded through fp16, tokens U(0,1)), upstream gradient N(0,1).

Prints ONE JSON line.  `value` is algorithmic bytes per second for the whole
step (forward 3 tensors + backward 5 tensors = 8*B*D*T*sizeof(dtype) bytes).
`roofline` describes the dominant kernel (the backward scan) from HIP-event
timings taken inside the timed region; `cpu_baseline` times the torch tree
scan (oracle/ref_scan.py, the restatement of the reference's ref.scan) on the
host cores on a bounded sample of the same workload.

`roofline.device_ceiling` is what a kernel without arithmetic reaches on the
same buffers with the same read/write mix (tests/native/stream_probe.hip),
timed after the scan's timed region.

Other workloads: --dtype {fp32,bf16,fp16,c64} --shape B D T; --gate {sigmoid,exp,lerp,
exp_norm} times the scans whose gate non-linearity (and, for lerp and exp_norm, whose
token) is formed inside the kernels: the first input then holds gate pre-activations
(logarithms for exp and exp_norm) of the same gates, the forward kernel moves 3 tensors
and the backward kernel 5 (sigmoid, exp) or 6 (lerp, exp_norm: it reads the values
again).  --reverse times the reverse scan and its own backward kernel.  --sweep FILE runs
the reference's benchmark grid, one JSON line per point into FILE and the same
points as a Markdown table into FILE.md and the (8,1536,T) grid as FILE.<direction>.csv (the
single summary line is still printed).  The reference's max-abs-error table is asserted by
tests/test_precision_gpu.py.
"""

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (ROOT, ROOT / "accelerated-scan_amd"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the backward kernel, from two rocprofv3 --pmc runs
# (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 KiB, factors from a plain copy of
# known size; summaries in profiles/).  Counters cannot be read from inside
# this script, so the figure is carried over from those runs, not measured in
# the run that prints it; `traffic_source` in the output says so.
MEASURED_TRAFFIC_BYTES = {
    ((8, 1536, 65536), "fp32"): 16134601632,  # FETCH_SIZE 4 729 483, WRITE_SIZE 6 297 835 KiB per dispatch
    ((8, 1536, 65536), "bf16"): 8070736352,   # FETCH_SIZE 2 366 349, WRITE_SIZE 3 149 061
}
TRAFFIC_SOURCE = {
    ((8, 1536, 65536), "fp32"): "profiles/scan_f32_8x1536x65536_fwd_bwd.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE); "
                                "not measured in this run",
    ((8, 1536, 65536), "bf16"): "profiles/scan_bf16_8x1536x65536_fwd_bwd.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE); "
                                "not measured in this run",
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 20; 200 for workloads below 1 GiB per tensor)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed warm-up steps (default 5; 100 for workloads below 1 GiB per tensor)")
    ap.add_argument("--dtype", choices=["fp32", "bf16", "fp16", "c64"], default="fp32")
    ap.add_argument("--shape", type=int, nargs=3, default=[8, 1536, 65536], metavar=("B", "D", "T"))
    ap.add_argument("--gate", choices=["identity", "sigmoid", "exp", "lerp", "exp_norm"], default="identity",
                    help="gate non-linearity applied inside the kernels (real dtypes; default: finished gates, "
                         "the reference's operator)")
    ap.add_argument("--reverse", action="store_true",
                    help="time the reverse scan x[t] = gate[t] x[t+1] + token[t] and its own fused backward kernel")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="for rocprofv3 --pmc runs: 3 plain copies of 1 GiB (torch copy_), then 3 steps "
                         "of the workload, no timing; the copy's known traffic scales the counters")
    ap.add_argument("--sweep", type=str, default=None, metavar="FILE",
                    help="also run the reference's benchmark grid ((8,1536,T), T=128..65536, forward / "
                         "reverse / backward / train, fp32 and bf16; complex (1,512,131072)) into FILE")
    return ap.parse_args()


GATE_CODES = {"identity": 0, "sigmoid": 1, "lerp": 2, "exp": 3, "exp_norm": 4}  # ascan_gate of include/ascan.h
GATES_WITH_VALUES = ("lerp", "exp_norm")


def make_inputs(shape, dtype_name, device, gate="identity"):
    import torch

    torch.manual_seed(12312323)
    if dtype_name == "c64":
        angle = 2 * torch.pi * torch.rand(*shape, device=device)
        radius = 0.9 + 0.1 * torch.rand(*shape, device=device)
        gates = torch.polar(radius, angle)
        tokens = torch.complex(torch.randn(*shape, device=device), torch.randn(*shape, device=device))
        grad_out = torch.complex(torch.randn(*shape, device=device), torch.randn(*shape, device=device))
        return gates, tokens, grad_out
    dt = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[dtype_name]
    gates = (0.999 + 0.001 * torch.rand(*shape, device=device)).half().float()
    if gate in ("sigmoid", "lerp"):  # the pre-activations of the same gates
        gates = torch.logit(gates.clamp(max=1.0 - 2.0 ** -20))
    elif gate in ("exp", "exp_norm"):  # their logarithms (strictly negative for exp_norm)
        gates = torch.log(gates).clamp(max=-(2.0 ** -20))
    tokens = torch.rand(*shape, device=device)
    grad_out = torch.randn(*shape, device=device)
    return gates.to(dt), tokens.to(dt), grad_out.to(dt)


def run_workload(shape, dtype_name, steps, warmup, gate="identity", reverse=False):
    """Times `steps` forward+backward passes; returns a dict of measurements.

    Tensors below 1 GiB are comparable to the 256 MB Infinity Cache, so such
    workloads rotate over four independent sets of buffers: step i scans set
    i forward and set i+2 backward, which puts more than a full step of other
    traffic between two uses of any buffer.  The headline tensors (3.2 GB each)
    need no rotation."""
    import torch

    from accelerated_scan import _abi

    device = torch.device("cuda:0")
    gates, tokens, grad_out = make_inputs(shape, dtype_name, device, gate)
    code = GATE_CODES[gate]
    bwd_tensors = 6 if gate in GATES_WITH_VALUES else 5

    def forward(g, x, states):
        if gate == "identity":
            _abi.forward(g, x, states, reverse)
        else:
            _abi.forward_gated(g, x, states, code)

    def backward(g, x, states, d, d_gates, d_tokens):
        if gate == "identity":
            _abi.backward(g, states, d, d_gates, d_tokens, reverse=reverse)
        elif gate in GATES_WITH_VALUES:
            _abi.backward_gated_values(g, x, states, d, d_gates, d_tokens, code)
        else:
            _abi.backward_gated(g, states, d, d_gates, d_tokens, code)

    elems = tokens.numel()
    esize = tokens.element_size()
    nsets = 1 if elems * esize >= (1 << 30) else 4
    sets = []
    for k in range(nsets):
        g, x, d = (gates, tokens, grad_out) if k == 0 else (gates.clone(), tokens.clone(), grad_out.clone())
        states, d_gates, d_tokens = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
        forward(g, x, states)  # the backward passes read valid states from the first step on
        sets.append((g, x, d, states, d_gates, d_tokens))

    def step(i, events=None):
        g, x, _, states, _, _ = sets[i % nsets]
        if events is not None:
            events[0].record()
        forward(g, x, states)
        if events is not None:
            events[1].record()
        g, x, d, states, d_gates, d_tokens = sets[(i + nsets // 2) % nsets]
        backward(g, x, states, d, d_gates, d_tokens)
        if events is not None:
            events[2].record()

    for i in range(warmup):
        step(i)
    # HIP events around each kernel, on the stream the kernels are launched on
    # (torch's current stream).  An event record costs about 5 us of stream time,
    # which is nothing beside the headline's 4.4 ms step but 3-4 % of a 0.4 ms
    # one: workloads below 1 GiB per tensor carry them on every fourth step.
    stride = 1 if nsets == 1 else 4
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] if i % stride == 0 else None
           for i in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(warmup + i, evs[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    sampled = [e for e in evs if e is not None]
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in sampled) / len(sampled)
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in sampled) / len(sampled)
    ms_per_step = (t1 - t0) * 1e3 / steps
    return {
        "buffers": sets,
        "elems": elems,
        "esize": esize,
        "input_sets": nsets,
        "event_steps": len(sampled),
        "ms_per_step": ms_per_step,
        "fwd_ms": fwd_ms,
        "bwd_ms": bwd_ms,
        "bwd_tensors": bwd_tensors,
        "gbps": (3 + bwd_tensors) * elems * esize / (ms_per_step * 1e-3) / 1e9,
        "fwd_gbps": 3 * elems * esize / (fwd_ms * 1e-3) / 1e9,
        "bwd_gbps": bwd_tensors * elems * esize / (bwd_ms * 1e-3) / 1e9,
    }


def load_stream_probe():
    """The no-arithmetic streaming kernels (tests/native/stream_probe.hip), or None
    when the probe library has not been built."""
    import ctypes

    path = ROOT / "tests" / "native" / "libstream_probe.so"
    if not path.exists():
        return None
    lib = ctypes.CDLL(str(path))
    lib.stream_probe_launch.restype = ctypes.c_int
    lib.stream_probe_launch.argtypes = ([ctypes.c_void_p] * 5 + [ctypes.c_int64] * 2 + [ctypes.c_int] * 5
                                        + [ctypes.c_uint, ctypes.c_void_p])
    lib.stream_probe_sweep.restype = ctypes.c_int
    lib.stream_probe_sweep.argtypes = ([ctypes.c_void_p] * 5 + [ctypes.c_int64] * 2 + [ctypes.c_int] * 4
                                       + [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint, ctypes.c_void_p])
    return lib


def device_ceiling(shape, dtype_name, bufs, steps=12, warmup=4):
    """Streams the workload's own buffers (`bufs`: the buffer sets of run_workload) with kernels that do no arithmetic:
    the backward scan's mix (3 tensors read, 2 written) and the forward scan's
    (2 read, 1 written), as a linear sweep of fresh workgroups, as one workgroup
    walking each row, and as a sweep in 64 KiB tiles that persistent workgroups take
    by ticket -- without and with the wait of a scan that passes carries from tile
    to tile through global memory.  Returns GB/s per variant; run outside the scan's
    timed region."""
    import torch

    probe = load_stream_probe()
    if probe is None:
        return None
    rows = shape[0] * shape[1]
    row_bytes = shape[2] * bufs[0][0].element_size()
    turn = [0]  # like the scan's own steps, successive launches rotate over the buffer sets
    nbytes = rows * row_bytes
    stream = torch.cuda.current_stream().cuda_stream
    out = {"unit": "GB/s",
           "what": "kernels without arithmetic on the same buffers, 16-byte nontemporal accesses "
                   "(tests/native/stream_probe.hip): linear = consecutive workgroups move consecutive 16 KiB; "
                   "row_walk = one 1024-thread workgroup per row in 64 KiB tiles with one barrier per tile, "
                   "the order of the scan kernels that own whole rows; ticket_sweep = one persistent 1024-thread "
                   "workgroup per compute unit takes 64 KiB tiles in memory order from a ticket counter, the order of "
                   "the scan kernels that pass carries through a table; ticket_sweep_carry_wait = the same, each "
                   "tile storing only after its row's earlier tiles have flagged their loads as landed"}
    for name, reads, writes, pattern in (("3R2W_linear", 3, 2, 0), ("3R2W_row_walk", 3, 2, 2),
                                         ("2R1W_linear", 2, 1, 0), ("2R1W_row_walk", 2, 1, 2)):
        def fn():
            g, x, d, states, d_gates, d_tokens = bufs[turn[0] % len(bufs)]
            turn[0] += 1
            rc = probe.stream_probe_launch(g.data_ptr(), states.data_ptr(), d.data_ptr(), d_gates.data_ptr(),
                                           d_tokens.data_ptr(), rows, row_bytes, reads, writes, pattern, 4, 1, 0, stream)
            if rc != 0:
                raise RuntimeError(f"stream probe: status {rc}")
        if (pattern == 0 and nbytes % (16 * 1024)) or (pattern != 0 and row_bytes % (64 * 1024)):
            out[name] = None  # the probe covers whole chunks / tiles only
            continue
        ms = time_call(fn, steps, warmup, min_ms=30.0)
        out[name] = (reads + writes) * nbytes / ms / 1e6
    tile = 64 * 1024
    if row_bytes % tile == 0 and row_bytes // tile <= 64 and rows * (row_bytes // tile) < 2 ** 31:
        table = torch.zeros(64 + rows * (row_bytes // tile) * 64, dtype=torch.uint8, device=bufs[0][0].device)
        grid = torch.cuda.get_device_properties(bufs[0][0].device).multi_processor_count
        for name, reads, writes, chain in (("3R2W_ticket_sweep", 3, 2, 0), ("3R2W_ticket_sweep_carry_wait", 3, 2, 1),
                                           ("2R1W_ticket_sweep", 2, 1, 0), ("2R1W_ticket_sweep_carry_wait", 2, 1, 1)):
            def fn():
                g, x, d, states, d_gates, d_tokens = bufs[turn[0] % len(bufs)]
                turn[0] += 1
                table.zero_()  # the scan's own launches clear their table too
                rc = probe.stream_probe_sweep(g.data_ptr(), states.data_ptr(), d.data_ptr(), d_gates.data_ptr(),
                                              d_tokens.data_ptr(), rows, row_bytes, reads, writes, chain, 4,
                                              table.data_ptr(), table.numel(), grid, stream)
                if rc != 0:
                    raise RuntimeError(f"stream probe: status {rc}")
            ms = time_call(fn, steps, warmup, min_ms=30.0)
            out[name] = (reads + writes) * nbytes / ms / 1e6
        torch.cuda.synchronize()
        if int(table[8:12].view(torch.int32).item()) != 0:
            raise RuntimeError("stream probe: a wait of the ticket sweep ran out")
    return out


def time_call(fn, steps, warmup, min_ms=0.0):
    """Mean milliseconds per call of fn() from HIP events on the current stream.
    With min_ms, short calls are repeated until the timed region lasts about that
    long (and the warm-up half as long): a handful of microsecond-sized launches
    is over before the clocks have settled."""
    import torch

    def timed(n):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(n):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / n

    for _ in range(warmup):
        fn()
    per_call = timed(steps)
    if min_ms > 0.0 and per_call * steps < min_ms:
        n = min(20000, int(min_ms / max(per_call, 1e-4)) + 1)
        timed(n // 2)
        per_call = timed(n)
    return per_call


def run_sweep(path, steps, warmup):
    """The reference's benchmark grid (tests/bench.py:14-31,100-115 of the
    reference): (8, 1536, T) for T = 128..65536, directions forward, reverse
    ("backward" in the reference's naming: a reverse forward scan, bench.py:75-77),
    fused backward, and train (autograd forward + backward including output
    allocation, bench.py:79-81; T <= 16384 as there); fp32 and bf16.  Then the
    complex forward + backward point of tests/bench_complex.py:79-90,
    (1, 512, 131072).  One JSON line per point."""
    import torch

    from accelerated_scan import _abi
    from accelerated_scan.complex import scan as complex_scan
    from accelerated_scan.warp import scan as warp_scan

    device = torch.device("cuda:0")
    min_ms = 40.0  # each point: at least 20 ms of warm-up and 40 ms timed (the reference warms up for seconds per point)
    records = []
    with open(path, "w") as f:
        def emit(rec):
            records.append(rec)
            f.write(json.dumps(rec) + "\n")
            f.flush()

        for dt in ("fp32", "bf16"):
            for T in [2 ** i for i in range(7, 17)]:
                shape = (8, 1536, T)
                gates, tokens, grad_out = make_inputs(shape, dt, device)
                out, d_gates, d_tokens = (torch.empty_like(tokens) for _ in range(3))
                nbytes = tokens.numel() * tokens.element_size()
                rec = {"dtype": dt, "shape": list(shape)}
                ms = time_call(lambda: _abi.forward(gates, tokens, out, False), steps, warmup, min_ms)
                rec["forward_ms"], rec["forward_GBps"] = ms, 3 * nbytes / ms / 1e6
                ms = time_call(lambda: _abi.forward(gates, tokens, out, True), steps, warmup, min_ms)
                rec["reverse_ms"], rec["reverse_GBps"] = ms, 3 * nbytes / ms / 1e6
                _abi.forward(gates, tokens, out, False)
                ms = time_call(lambda: _abi.backward(gates, out, grad_out, d_gates, d_tokens), steps, warmup, min_ms)
                rec["backward_ms"], rec["backward_GBps"] = ms, 5 * nbytes / ms / 1e6
                if T <= 16384:
                    g = gates.clone().requires_grad_(True)
                    x = tokens.clone().requires_grad_(True)
                    ms = time_call(lambda: torch.autograd.grad(warp_scan(g, x), (g, x), grad_out), steps, warmup, min_ms)
                    rec["train_ms"], rec["train_GBps"] = ms, 8 * nbytes / ms / 1e6
                    if T <= 2048:  # where the host cost shows: the same with the process on one core
                        with one_core():
                            ms = time_call(lambda: torch.autograd.grad(warp_scan(g, x), (g, x), grad_out), steps, warmup,
                                           min_ms)
                        rec["train_one_core_ms"], rec["train_one_core_GBps"] = ms, 8 * nbytes / ms / 1e6
                        # and with the backward pass run by the calling thread instead of autograd's device thread
                        torch.autograd.set_multithreading_enabled(False)
                        try:
                            ms = time_call(lambda: torch.autograd.grad(warp_scan(g, x), (g, x), grad_out), steps, warmup,
                                           min_ms)
                        finally:
                            torch.autograd.set_multithreading_enabled(True)
                        rec["train_one_thread_ms"], rec["train_one_thread_GBps"] = ms, 8 * nbytes / ms / 1e6
                    del g, x
                # forward + backward captured once into a HIP graph and replayed: what a caller reaches who
                # takes the per-call host cost (Python, autograd, allocation) out of the loop
                ms = time_call(graphed_step(gates, tokens, grad_out, out, d_gates, d_tokens), steps, warmup, min_ms)
                rec["train_graph_ms"], rec["train_graph_GBps"] = ms, 8 * nbytes / ms / 1e6
                emit(rec)
                del gates, tokens, grad_out, out, d_gates, d_tokens

        shape = (1, 512, 131072)
        gates, tokens, grad_out = make_inputs(shape, "c64", device)
        out, d_gates, d_tokens = (torch.empty_like(tokens) for _ in range(3))
        nbytes = tokens.numel() * tokens.element_size()

        def both():
            _abi.forward(gates, tokens, out, False)
            _abi.backward(gates, out, grad_out, d_gates, d_tokens)

        ms = time_call(both, steps, warmup, min_ms)
        rec = {"dtype": "c64", "shape": list(shape), "forward_backward_ms": ms,
               "forward_backward_GBps": 8 * nbytes / ms / 1e6}
        g = gates.clone().requires_grad_(True)
        x = tokens.real.contiguous().requires_grad_(True)  # real inputs, as the reference's complex bench
        ms = time_call(lambda: torch.autograd.grad(complex_scan(g, x), (g, x), grad_out), steps, warmup, min_ms)
        rec["train_real_inputs_ms"] = ms
        emit(rec)
    write_sweep_markdown(records, str(path) + ".md", steps, warmup)
    write_sweep_csv(records, str(path))


class one_core:
    """Pins every thread of this process to one of its cores for the duration.  A decode-sized
    autograd step is a hand-over between the calling thread and autograd's backward thread (and the
    HIP runtime's own threads); on these virtual hosts a wake-up across cores costs tens of
    microseconds in some processes and not in others, and a process confined to one core
    (`taskset -c N python ...` does the same from outside) never pays it."""

    def __enter__(self):
        self.allowed = os.sched_getaffinity(0)
        self.threads = [int(t) for t in os.listdir("/proc/self/task")]
        core = {sorted(self.allowed)[0]}
        for t in self.threads:
            try:
                os.sched_setaffinity(t, core)
            except OSError:
                pass  # a thread that ended meanwhile
        return self

    def __exit__(self, *exc):
        for t in self.threads:
            try:
                os.sched_setaffinity(t, self.allowed)
            except OSError:
                pass
        return False


def graphed_step(gates, tokens, grad_out, out, d_gates, d_tokens):
    """Captures one forward + backward through the C ABI (outputs and tables allocated
    beforehand) into a HIP graph; returns the function that replays it."""
    import torch

    from accelerated_scan import _abi

    rows, seqlen, code = _abi._problem(gates, tokens)
    nbytes = _abi.load().ascan_workspace_bytes(rows, seqlen, code)
    tables = [torch.empty(nbytes, dtype=torch.uint8, device=gates.device) if nbytes else None for _ in range(2)]

    def step():
        _abi.forward(gates, tokens, out, False, workspace=tables[0])
        _abi.backward(gates, out, grad_out, d_gates, d_tokens, workspace=tables[1])

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    return graph.replay


SWEEP_DIRECTIONS = ("forward", "reverse", "backward", "train", "train_one_core", "train_one_thread", "train_graph")


def write_sweep_csv(records, stem):
    """The (8, 1536, T) grid as CSV, one file per direction (STEM.<direction>.csv) with a
    SEQUENCE_LENGTH column and one column of milliseconds per dtype, as the reference's
    harness saves them (tests/bench.py:100-115 of the reference); empty cells were not measured."""
    dtypes = [dt for dt in ("fp32", "bf16") if any(r["dtype"] == dt for r in records)]
    lengths = sorted({r["shape"][2] for r in records if r["dtype"] in dtypes})
    for direction in SWEEP_DIRECTIONS:
        with open(f"{stem}.{direction}.csv", "w") as f:
            f.write("SEQUENCE_LENGTH," + ",".join(f"{dt}_ms" for dt in dtypes) + "\n")
            for T in lengths:
                cells = []
                for dt in dtypes:
                    rec = next((r for r in records if r["dtype"] == dt and r["shape"][2] == T), {})
                    cells.append(f"{rec[direction + '_ms']:.6f}" if direction + "_ms" in rec else "")
                f.write(f"{T}," + ",".join(cells) + "\n")


def write_sweep_markdown(records, path, steps, warmup):
    """The sweep as a table: ms per call and algorithmic TB/s (3 tensors forward /
    reverse, 5 backward, 8 train)."""
    import hashlib

    # identifies the kernels measured wherever the file is written (the GPU box has no git checkout):
    # sha1 over the library's sources in name order
    digest = hashlib.sha1()
    for src in sorted(list((ROOT / "accelerated-scan_amd" / "csrc").glob("*.h*")) + [ROOT / "include" / "ascan.h"]):
        digest.update(src.name.encode() + b"\0" + src.read_bytes())
    head = digest.hexdigest()[:12]
    def cell(rec, key):
        if f"{key}_ms" not in rec:
            return "—"
        return f"{rec[f'{key}_ms']:.4f} ({rec[f'{key}_GBps'] / 1e3:.2f})"

    with open(path, "w") as f:
        f.write("# Scan sweep on MI355X: the reference's benchmark grid (tests/bench.py:14-31 of the reference)\n\n")
        f.write(f"Generated by `python bench.py --sweep FILE` (sha1 of csrc/* and include/ascan.h in name order: {head}; mean over at "
                f"least {steps} calls and 40 ms after at least {warmup} calls and 20 ms of warm-up, HIP events; one set of buffers per point, so tensors up to a few hundred MB "
                "see some Infinity Cache hits). Cells: ms per call (algorithmic TB/s). forward / reverse / backward "
                "are kernel calls through the C ABI; train = autograd forward + backward of `warp.scan`, "
                "allocation included; train (one core) = the same with every thread of the process pinned to one core "
                "(T <= 2048, where the host cost shows: on these virtual hosts the hand-over between the calling thread "
                "and autograd's backward thread costs tens of microseconds across cores in some processes, none on one "
                "core; `taskset -c N` from outside does the same); train (one thread) = the same with "
                "`torch.autograd.set_multithreading_enabled(False)`, which runs the backward pass on the calling thread "
                "and takes the hand-over away; train (graph) = forward + backward through the C ABI "
                "captured once into a HIP graph and replayed, i.e. without the per-call host cost.\n")
        for dt in ("fp32", "bf16"):
            f.write(f"\n## {dt}, shape (8, 1536, T)\n\n| T | forward | reverse | backward | train | train (one core) | "
                    "train (one thread) | train (graph) |\n|---|---|---|---|---|---|---|---|\n")
            for rec in records:
                if rec["dtype"] == dt:
                    f.write(f"| {rec['shape'][2]} | {cell(rec, 'forward')} | {cell(rec, 'reverse')} | "
                            f"{cell(rec, 'backward')} | {cell(rec, 'train')} | {cell(rec, 'train_one_core')} | "
                            f"{cell(rec, 'train_one_thread')} | {cell(rec, 'train_graph')} |\n")
        for rec in records:
            if rec["dtype"] == "c64":
                f.write(f"\n## complex64, shape {tuple(rec['shape'])} (tests/bench_complex.py:79-90 of the reference)\n\n"
                        f"forward + backward through the C ABI: {rec['forward_backward_ms']:.4f} ms "
                        f"({rec['forward_backward_GBps'] / 1e3:.2f} TB/s); autograd forward + backward with real "
                        f"inputs: {rec['train_real_inputs_ms']:.4f} ms\n")


def cpu_baseline(shape, dtype_name):
    """Tree scan (the reference's CPU path, restated) forward+backward on the
    host cores, on a slice of the workload's rows sized to take ~10-30 s."""
    import torch

    from oracle import ref_scan

    B, D, T = shape
    rows = max(1, min(B * D, (3 << 27) // T))  # about 400M elements per repetition: ~3 s each on 16 cores
    sample = (1, rows, T)
    gates, tokens, grad_out = make_inputs(sample, dtype_name, torch.device("cpu"))
    if dtype_name in ("bf16", "fp16"):
        gates, tokens, grad_out = gates.float(), tokens.float(), grad_out.float()

    def once():
        g = gates.clone().requires_grad_(True)
        x = tokens.clone().requires_grad_(True)
        t0 = time.perf_counter()
        out = ref_scan.scan(g, x)
        torch.autograd.grad(out, (g, x), grad_out)
        return time.perf_counter() - t0

    once()  # warm-up
    times = sorted(once() for _ in range(3))
    median = times[1]
    esize = 8 if dtype_name == "c64" else 4
    return {
        "value": 8 * rows * T * esize / median / 1e9,
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"torch tree scan fwd+bwd (autograd), fp32 arithmetic, shape {sample} "
                  f"= {rows} of {B * D} rows, median of 3: {median * 1e3:.1f} ms; "
                  f"host has {os.cpu_count()} logical cpus",
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (rows shard without communication); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 2
    from accelerated_scan import _abi

    if not _abi.library_path().exists():  # normally built beforehand; build only when nothing is there
        import __graft_entry__

        __graft_entry__.build()
    _abi.load()  # no fallback: fail here if the HIP library is missing

    shape = tuple(args.shape)
    gated = args.gate != "identity"
    if gated and args.dtype == "c64":
        print("bench.py: --gate needs a real dtype", file=sys.stderr)
        return 2
    if gated and args.reverse:
        print("bench.py: the gated scans run forward in time only", file=sys.stderr)
        return 2
    # Sub-millisecond steps need a longer run: with 5 + 20 steps of 0.4 ms the whole measurement is over in 10 ms,
    # before clocks and caches have settled (measured at (4,1024,8192) complex64: 68.4 % of peak with 5 + 20 steps,
    # 72.2 % with 100 + 200).  The headline's defaults are the driver's: 5 + 20 steps of 4.4 ms.
    tensor_bytes = shape[0] * shape[1] * shape[2] * {"fp32": 4, "bf16": 2, "fp16": 2, "c64": 8}[args.dtype]
    small = tensor_bytes < (1 << 30)
    if args.steps is None:
        args.steps = 200 if small else 20
    if args.warmup is None:
        args.warmup = 100 if small else 5
    if args.pmc_calibration:
        src = torch.rand(1 << 28, device="cuda:0")  # 1 GiB of fp32
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        m = run_workload(shape, args.dtype, 3, 0, args.gate, args.reverse)
        device_ceiling(shape, args.dtype, m["buffers"], steps=3, warmup=0)  # the probe kernels, for the same counters
        print(json.dumps({"calibration_copy_bytes_read": src.numel() * 4, "calibration_copy_bytes_written":
                          src.numel() * 4, "workload_shape": list(shape), "dtype": args.dtype}))
        return 0
    m = run_workload(shape, args.dtype, args.steps, args.warmup, args.gate, args.reverse)
    ceiling = device_ceiling(shape, args.dtype, m.pop("buffers"))

    if args.sweep:
        run_sweep(args.sweep, 20, 5)

    dtype_field = {"fp32": "f32", "bf16": "bf16 storage, f32 arithmetic",
                   "fp16": "f16 storage, f32 arithmetic", "c64": "complex64 (f32 pairs)"}[args.dtype]
    bwd_bytes = m["bwd_tensors"] * m["elems"] * m["esize"]
    gate_text = {"identity": "", "sigmoid": ", gates = sigmoid(stored) inside the kernels",
                 "exp": ", gates = exp(stored) inside the kernels",
                 "lerp": ", x[t] = a x[t-1] + (1 - a) v[t] with a = sigmoid(stored) inside the kernels",
                 "exp_norm": ", x[t] = a x[t-1] + sqrt(1 - a^2) v[t] with a = exp(stored) inside the kernels"}[args.gate]
    result = {
        "metric": f"fwd+bwd achieved HBM GB/s (algorithmic bytes: 3 tensors forward + {m['bwd_tensors']} backward) "
                  f"at {shape} {args.dtype}" + gate_text + (", reverse scan and its backward pass" if args.reverse else ""),
        "value": m["gbps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_field,
        "data": "synthetic",
        "config": {
            "workload": ("reverse scan + its fused backward" if args.reverse else "scan forward + fused backward")
                        + f", shape {list(shape)}, {args.dtype}, " + (
                "gates r*exp(i*theta) with r ~ 0.9+0.1*U(0,1), tokens and grad_out complex N(0,1)"
                if args.dtype == "c64" else "gates 0.999+0.001*U(0,1), tokens U(0,1), grad_out N(0,1)") + (
                f"; gate {args.gate}: the first input holds the gates' " + (
                    "logarithms" if args.gate in ("exp", "exp_norm") else "sigmoid pre-activations") if gated else ""),
            "input_sets": m["input_sets"],
            "steps_with_kernel_events": m["event_steps"],
            "fwd_ms": m["fwd_ms"],
            "bwd_ms": m["bwd_ms"],
            "fwd_GBps": m["fwd_gbps"],
            "bwd_GBps": m["bwd_gbps"],
            "frac_of_hbm_peak": m["gbps"] / HBM_PEAK_GBPS,
        },
        "roofline": {
            "kernel": "scan_backward_kernel",
            "bound": "hbm",
            "achieved": m["bwd_gbps"],
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": m["bwd_gbps"] / HBM_PEAK_GBPS,
            "algorithmic_bytes_per_launch": bwd_bytes,
            "avg_launch_ms": m["bwd_ms"],
            "traffic": None if gated else MEASURED_TRAFFIC_BYTES.get((shape, args.dtype)),
            "traffic_source": None if gated else TRAFFIC_SOURCE.get((shape, args.dtype)),
            "device_ceiling": ceiling,
        },
    }
    if not args.no_cpu_baseline and not gated and not args.reverse:  # the baseline is the reference's operator
        result["cpu_baseline"] = cpu_baseline(shape, args.dtype)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
