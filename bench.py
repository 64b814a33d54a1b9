#!/usr/bin/env python3
"""Benchmark of the NeuZip codec hot path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the
fused rANS-decode + merge kernel reconstructing a batch of R = 5 bf16 weights
of 16384 x 4096 values N(0, 0.02) each (lossless, 7 mantissa bits kept; five
seeds) from their compressed form, one launch per weight, everything resident
in HBM.  Five independent weights, because one of them (223 MB of compressed
input plus dense output) fits the 256 MB last-level cache and would be served
from there when decoded over and over.

Prints ONE JSON line:
  value          dense bf16 bytes produced per second (R * 2N / step), GB/s
  roofline       algorithmic bytes of one decode launch (C + P + 2N) over its
                 mean duration (HIP events on the launch stream) vs 8 TB/s,
                 measured on the rotation (= roofline_cold)
  roofline_hot   the same kernel on one weight decoded repeatedly (cache-resident)
  stress_8192x28672  BASELINE config 5 (448 MiB dense), precision 7 and 3
  sweep          decode/encode throughput and stored size for 7/3/1/0 kept bits
  cpu_baseline   the CPU oracle (same container format) timed on the host cores
  llama8b_shape  tokens/s of the 8B-shaped decoder with compressed weights: the
                 unchanged caller (import neuzip; Manager(precision=7).convert)
                 first, the package's extensions beside it
  gpt2m_shape    BASELINE config 4: 20 timed AdamW steps of a GPT-2-medium-shaped
                 model with its weights kept compressed, against dense
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


STRESS_ROWS, STRESS_COLS = 8192, 28672  # BASELINE config 5
PROFILE_DIR = os.path.join(ROOT, "profiles")


def recorded_traffic(key: str):
    """HBM bytes one launch moved according to rocprofv3 counters, as recorded in a
    summary under profiles/ (a line ``traffic_bytes_per_launch[<key>] = <bytes>``; a
    live run cannot read the counters).  -> (bytes, "profiles/<file>") or (None, None)."""
    import glob
    import re

    for path in sorted(glob.glob(os.path.join(PROFILE_DIR, "*.txt"))):
        try:
            text = open(path).read()
        except OSError:
            continue
        for k, v in re.findall(r"traffic_bytes_per_launch\[(.*?)\]\s*=\s*(\d+)", text):
            if k.strip() == key:
                return int(v), "profiles/" + os.path.basename(path)
    return None, None


def roofline_block(algo_bytes, launch_s, precision, working_set, launches, note=None):
    achieved = algo_bytes / launch_s / 1e9
    blk = {
        "bound": "hbm",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": None,
        "kernel": f"nz_decode_kernel<{precision}>",
        "algorithmic_bytes_per_launch": int(algo_bytes),
        "mean_launch_us": round(launch_s * 1e6, 2),
        "launches_timed": launches,
        "working_set_bytes": int(working_set),
    }
    if note:
        blk["note"] = note
    return blk


def normal_weight(torch, rows, cols, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(rows, cols, device="cuda", generator=g) * 0.02).to(torch.bfloat16).view(-1)


def stress_weight(torch, rows, cols, seed):
    """BASELINE config 5: Student-t(3) x 0.02, 16 outlier columns x 50, 1 % exact zeros,
    0.1 % subnormals (random sign and mantissa, exponent 0)."""
    g = torch.Generator(device="cuda").manual_seed(seed + 1000)
    z = torch.randn(rows, cols, device="cuda", generator=g)
    chi = sum(torch.randn(rows, cols, device="cuda", generator=g) ** 2 for _ in range(3)) / 3.0
    x = z / chi.sqrt() * 0.02
    del z, chi
    cols_out = torch.randperm(cols, device="cuda", generator=g)[:16]
    x[:, cols_out] *= 50.0
    w = x.to(torch.bfloat16).view(-1)
    del x
    r = torch.rand(rows * cols, device="cuda", generator=g)
    bits = w.view(torch.int16)
    bits[r < 0.01] = 0
    sub = (r >= 0.01) & (r < 0.011)
    k = int(sub.sum())
    mant = torch.randint(1, 128, (k,), device="cuda", generator=g, dtype=torch.int16)
    sign = torch.randint(0, 2, (k,), device="cuda", generator=g, dtype=torch.int16) * torch.tensor(-32768, dtype=torch.int16, device="cuda")
    bits[sub] = mant | sign
    return w


def closed_form_torch(torch, dense, s):
    """What the reference returns for the bf16 values `dense` at precision s, as int16 bit
    patterns: the 15-bit magnitude rounded half-up to a multiple of 2^(7-s), modulo 2^15."""
    bits = dense.view(torch.int16)
    if s == 7:
        return bits
    v = bits.to(torch.int32) & 0xFFFF
    mag = ((v & 0x7FFF) + (1 << (6 - s))) & 0x7FFF & (0x7FFF ^ ((1 << (7 - s)) - 1))
    out = (v & 0x8000) | mag
    return torch.where(out >= 32768, out - 65536, out).to(torch.int16)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rows", type=int, default=16384)
    ap.add_argument("--cols", type=int, default=4096)
    ap.add_argument("--precision", type=int, default=7, choices=[7, 3, 1, 0])
    ap.add_argument("--chunk-size", type=int, default=0,
                    help="elements per frequency table; 0 = library default (131072), 65536 = the reference's nvcomp chunk")
    ap.add_argument("--lane-symbols", type=int, default=None,
                    help="0 = library default; -1 = chosen per tensor (the default of the model workloads)")
    ap.add_argument("--size-budget", type=float, default=0.0,
                    help="model workloads: stored exponent bytes over their entropy that the per-tensor geometry "
                         "may spend (default: the library's 1.01; e.g. 1.04 buys wavefronts for small matrices)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--rotate", type=int, default=5,
                    help="independent stored copies of the workload a step decodes one after the other "
                         "(5 x 223 MB: out of the 256 MB last-level cache); 1 = one copy over and over")
    ap.add_argument("--settle-s", type=float, default=0.25,
                    help="seconds of untimed decode launches before the warm-up steps (clock settling)")
    ap.add_argument("--no-hot", action="store_true", help="skip the cache-resident single-tensor timing")
    ap.add_argument("--no-stress", action="store_true", help="skip the 8192x28672 stress tensor (BASELINE config 5)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--cpu-threads", type=int, default=0, help="0 = all host cores given to this process")
    ap.add_argument("--workload", default="tensor", choices=["tensor", "llama8b", "gpt2m"],
                    help="tensor: decode of one 16384x4096 weight (the headline metric); llama8b: 512-token "
                         "prompt + greedy decode on a Llama-3-8B-shaped model with compressed weights; "
                         "gpt2m: training steps on a GPT-2-medium-shaped model with compressed weights")
    ap.add_argument("--layers", type=int, default=0, help="override the layer count of the model workloads")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--decode-steps", type=int, default=128)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--seq-len", type=int, default=1024)
    ap.add_argument("--verify-steps", type=int, default=10,
                    help="gpt2m: steps of the side-by-side dense / compressed weight comparison")
    ap.add_argument("--no-gpt2m", action="store_true",
                    help="skip the GPT-2-medium-shaped training block (BASELINE config 4) of the default line")
    ap.add_argument("--no-llama", action="store_true",
                    help="skip the 8B-shaped decoder that the default run appends to the codec line")
    ap.add_argument("--encode-phases", action="store_true",
                    help="only print the encode kernel's time per phase (library built with -DNZ_PROBE_PHASES)")
    ap.add_argument("--protocol-probe", action="store_true",
                    help="only compare the timing protocols of a sweep point (see protocol_probe)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run five plain 256 MiB device copies (to scale FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


class Stored:
    """One compressed tensor: container and packed stream in buffers of their own."""

    __slots__ = ("comp", "packed", "total", "packed_bytes", "n", "s")


class Workspace:
    """Scratch and bound-sized staging shared by the stateless C-ABI calls of this run."""

    def __init__(self, torch, L, lib_mod, n_max, chunk, lane):
        self.torch, self.L, self.m = torch, L, lib_mod
        self.chunk, self.lane = chunk, lane
        cap = L.nz_exp_bound_bytes(n_max, chunk, lane)
        if cap == 0:
            raise SystemExit("unsupported chunk_size / lane_symbols combination")
        self.cap = int(cap)
        self.stage = torch.empty(self.cap, dtype=self.torch.uint8, device="cuda")
        self.ws_bytes = int(L.nz_encode_workspace_bytes(n_max, chunk, lane))
        self.ws = torch.empty(self.ws_bytes, dtype=self.torch.uint8, device="cuda")
        self.aux = torch.zeros(4, dtype=self.torch.int64, device="cuda")
        self.status = torch.zeros(2, dtype=self.torch.int32, device="cuda")

    def _encode(self, dense, s, packed, comp, cap, sync):
        st = self.torch.cuda.current_stream().cuda_stream
        total = ctypes.c_uint64(0)
        rc = self.L.nz_encode(dense.data_ptr(), dense.numel(), s, self.chunk, self.lane, packed.data_ptr(),
                              comp.data_ptr(), cap, self.ws.data_ptr(), self.ws_bytes, self.aux.data_ptr(),
                              self.aux.data_ptr() + 8, ctypes.byref(total) if sync else None, 0, None, st)
        if rc != 0:
            raise RuntimeError(self.m.last_error())
        return int(total.value)

    def encode(self, dense, s) -> Stored:
        """Compress `dense` into exact-size buffers of its own."""
        n = dense.numel()
        st = Stored()
        st.n, st.s = n, s
        st.packed_bytes = int(self.L.nz_packed_stored_bytes(n, s, self.chunk, self.lane))
        st.packed = self.torch.empty(max(8, st.packed_bytes), dtype=self.torch.uint8, device="cuda")
        st.total = self._encode(dense, s, st.packed, self.stage, self.cap, True)
        # room up to the bound, so that encode_into can write the same tensor again in place
        st.comp = self.torch.empty(int(self.L.nz_exp_bound_bytes(n, self.chunk, self.lane)), dtype=self.torch.uint8,
                                   device="cuda")
        st.comp[: st.total].copy_(self.stage[: st.total])
        return st

    def encode_into(self, dense, s, st: Stored) -> None:
        """The encode again, asynchronously, into the buffers of `st`."""
        self._encode(dense, s, st.packed, st.comp, st.comp.numel(), False)

    def decode(self, st: Stored, out, check=False, flags=0):
        stream = self.torch.cuda.current_stream().cuda_stream
        rc = self.L.nz_decode(st.comp.data_ptr(), st.total, st.packed.data_ptr(), st.n, st.s, self.chunk, self.lane,
                              out.data_ptr(), self.status.data_ptr(), (1 if check else 0) | flags, 0, None, stream)
        if rc != 0:
            raise RuntimeError(self.m.last_error())


def time_launches(torch, fn, steps, warmup):
    """`steps` back-to-back launches between two synchronisations: wall time on
    the host clock, and the time between two HIP events recorded on the launch
    stream right before the first and right after the last launch (nothing else
    is enqueued in between: an event record between two launches costs ~5 us
    and lets the GPU idle, after which a launch runs ~5 % slower).
    -> wall seconds, event seconds per launch."""
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) * 1e-3 / steps


def settled_launches(torch, fn, steps, warmup, settle_s):
    """time_launches after `settle_s` seconds of the same launches, untimed: every
    measured point of a run gets the settled clocks the headline gets.
    -> wall seconds, event seconds per launch, untimed launches"""
    n = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_s:
        fn()
        torch.cuda.synchronize()
        n += 1
    wall, per = time_launches(torch, fn, steps, warmup)
    return wall, per, n + warmup


def protocol_probe(args, torch, L, lib_mod):
    """Why a sweep point needs the headline's protocol.  For every precision,
    three times over: five weights encoded into fresh buffers (host-synchronised,
    as the sweep does), then their decode timed (a) the way the sweep used to -
    two warm-up steps, ten steps between the events - (b) the same after 0.2 s
    without work, (c) settled, twenty steps.  One JSON line per measurement;
    (a) once more per precision with an event after every step."""
    n, R = args.rows * args.cols, max(1, args.rotate)
    ws = Workspace(torch, L, lib_mod, n, lib_mod.DEFAULT_CHUNK, lib_mod.DEFAULT_LANE_SYMS)
    denses = [normal_weight(torch, args.rows, args.cols, args.seed + i) for i in range(R)]
    outs = [torch.empty_like(d) for d in denses]

    def point(s, k, settle_s, idle_s, per_step=False):
        ss = [ws.encode(d, s) for d in denses]

        def dec():
            for st, o in zip(ss, outs):
                ws.decode(st, o)

        torch.cuda.synchronize()
        if idle_s:
            time.sleep(idle_s)
        if per_step:
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(k + 1)]
            for _ in range(2):
                dec()
            evs[0].record()
            for i in range(k):
                dec()
                evs[i + 1].record()
            torch.cuda.synchronize()
            print(json.dumps({"precision": s, "protocol": "two warm-up steps, an event after every step",
                              "launch_us_per_step": [round(evs[i].elapsed_time(evs[i + 1]) * 1e3 / R, 1)
                                                     for i in range(k)]}), flush=True)
            return
        if settle_s:
            w, m, _ = settled_launches(torch, dec, k, 2, settle_s)
        else:
            w, m = time_launches(torch, dec, k, 2)
        print(json.dumps({"precision": s, "steps": k, "settle_s": settle_s, "idle_s_before": idle_s,
                          "launch_us": round(m / R * 1e6, 2), "decode_GBps": round(2 * n / (m / R) / 1e9, 1),
                          "wall_over_event": round(w / (m * k), 3)}), flush=True)

    for _ in range(3):
        for s in (7, 3, 1, 0):
            point(s, 10, 0, 0)
            point(s, 10, 0, 0.2)
            point(s, 20, args.settle_s / 2, 0)
    for s in (7, 3, 1, 0):
        point(s, 10, 0, 0, per_step=True)
    return 0


def encode_phases(args, torch, L, lib_mod):
    """Where the time of nz_encode_kernel goes, phase by phase.  Needs a library
    built with NZ_HIPCC_EXTRA=-DNZ_PROBE_PHASES (thread 0 of every workgroup then
    adds the shader-clock cycles between the phase boundaries to six counters)."""
    if not hasattr(L, "nz_probe_read") or args.precision != 7:
        print("needs a library built with -DNZ_PROBE_PHASES, and precision 7 (the counters sit in that "
              "precision's translation unit)", file=sys.stderr)
        return 2
    L.nz_probe_read.argtypes = [ctypes.POINTER(ctypes.c_ulonglong), ctypes.c_int]
    n = args.rows * args.cols
    chunk, lane = args.chunk_size or lib_mod.DEFAULT_CHUNK, args.lane_symbols or lib_mod.DEFAULT_LANE_SYMS
    ws = Workspace(torch, L, lib_mod, n, chunk, lane)
    dense = normal_weight(torch, args.rows, args.cols, args.seed)
    st = ws.encode(dense, args.precision)
    for _ in range(50):
        ws.encode_into(dense, args.precision, st)
    torch.cuda.synchronize()
    acc = (ctypes.c_ulonglong * 8)()
    L.nz_probe_read(acc, 1)
    k = max(100, args.steps)
    _, per = time_launches(torch, lambda: ws.encode_into(dense, args.precision, st), k, 0)
    L.nz_probe_read(acc, 0)
    names = ("split + histogram", "table", "coding", "finalize + announce", "wait for the chunks before", "record move")
    groups = k * (-(-n // chunk))
    total = float(sum(acc[i] for i in range(6)))
    print(json.dumps({
        "kernel": f"nz_encode_kernel<{args.precision}, *>", "rows": args.rows, "cols": args.cols, "chunk_size": chunk,
        "lane_symbols": lane, "launches": k, "launch_us": round(per * 1e6, 2),
        "cycles_per_workgroup": {nm: round(acc[i] / groups) for i, nm in enumerate(names)},
        "share": {nm: round(acc[i] / total, 4) for i, nm in enumerate(names)},
    }))
    return 0


def _timed(torch, fn):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = fn()
    torch.cuda.synchronize()
    return time.perf_counter() - t0, out


def entropy_bound_bytes(torch, exps, chunk=65536):
    """order-0 entropy of the exponent bytes `exps` (int32 on the device), per 64 Ki of them, in bytes"""
    n = exps.numel()
    nch = (n + chunk - 1) // chunk
    idx = torch.arange(n, device=exps.device, dtype=torch.int64) // chunk
    cnt = torch.bincount(idx * 256 + exps.to(torch.int64), minlength=256 * nch).view(nch, 256).double()
    p = cnt / cnt.sum(1, keepdim=True).clamp_min(1.0)
    h = -(torch.where(cnt > 0, cnt * torch.log2(p.clamp_min(1e-300)), torch.zeros_like(cnt))).sum()
    return float(h) / 8.0


def size_over_entropy(torch, mgr, precision, handles=None):
    """Bytes stored for the exponents of every entry (all that is held, less what
    the reference's packed sign|mantissa stream takes: the container keeps some
    of those bytes in its coder states) over the order-0 entropy bound of the
    stored exponents: over all entries together, and the largest single ratio
    with the shape and geometry it belongs to."""
    from neuzip_amd import _lib

    L = _lib.load()
    be = mgr._be
    exp_total, bound_total, worst = 0, 0.0, None
    geoms = {}
    for h in (handles or list(mgr.meta_dict)):
        w = mgr.read(h)
        exps = (w.view(torch.int16).reshape(-1).to(torch.int32) >> 7) & 0xFF
        bound = entropy_bound_bytes(torch, exps)
        n = int(w.numel())
        del w, exps
        eb = mgr.size(h) - int(L.nz_packed_bytes(n, precision))
        exp_total += eb
        bound_total += bound
        g = be.geometry(h)
        geoms[g] = geoms.get(g, 0) + 1
        if bound > 0 and (worst is None or eb / bound > worst[0]):
            worst = (eb / bound, list(mgr.meta_dict[h]), list(g))
    return {
        "all_entries": round(exp_total / bound_total, 5) if bound_total else None,
        "largest": None if worst is None else {"ratio": round(worst[0], 5), "shape": worst[1], "chunk_lane": worst[2]},
        "size_budget": round(be.size_budget, 4),
        "geometries_chunk_lane_count": sorted([list(g) + [c] for g, c in geoms.items()]),
    }


def make_manager(args, precision):
    """The manager of a model workload: with no geometry flags it is built exactly
    as a user of the reference builds it (``import neuzip;
    neuzip.Manager(precision=...)``); flags go through the package's own class."""
    if not args.chunk_size and args.lane_symbols in (-1, None) and not args.size_budget:
        import neuzip

        return neuzip.Manager(precision=precision), "import neuzip; neuzip.Manager(precision=%d)" % precision
    import neuzip_amd

    lane = "auto" if args.lane_symbols in (-1, None) else args.lane_symbols
    return (neuzip_amd.Manager(precision=precision, chunk_size=args.chunk_size or None, lane_symbols=lane,
                               size_budget=args.size_budget or None),
            f"neuzip_amd.Manager(precision={precision}, chunk_size={args.chunk_size or None}, lane_symbols={lane!r}, "
            f"size_budget={args.size_budget or None})")


def llama8b_measure(args, torch, full):
    """Llama-3-8B-shaped decoder, all Linear weights stored lossless-compressed,
    batch 1, 512-token prompt + 128 greedy steps, against the same model with
    dense weights.  Every mode runs the same static-cache decode step, eagerly
    or as a replayed HIP graph; compressed weights are decoded per Linear (the
    reference's granularity), or per transformer block with one launch, with or
    without decoding the next block ahead on a side stream, or not at all as a
    dense tensor (decode fused into the matrix-vector product).  The first
    compressed mode is the unchanged caller: the model converted with
    ``import neuzip; neuzip.Manager(precision=...).convert(model)`` and run as
    it is (its single-token Linears go through the fused product one by one).
    `full` adds the per-block modes."""
    import neuzip_amd
    from bench_models import LlamaShaped

    layers = args.layers or 32
    torch.manual_seed(args.seed)
    with torch.device("cuda"):
        torch.set_default_dtype(torch.bfloat16)
        model = LlamaShaped(layers=layers)
        torch.set_default_dtype(torch.float32)
    model.eval()
    T = args.prompt_len
    prompt = torch.randint(0, 128256, (1, T), device="cuda")
    steps = args.decode_steps
    kcs, vcs = model.static_caches(T + steps)
    tok_buf = torch.zeros(1, 1, dtype=torch.int64, device="cuda")
    pos_buf = torch.zeros(1, dtype=torch.int64, device="cuda")

    def sync_time(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, out

    def run_mode(graph, n_steps=None):
        """-> (prefill seconds, decode seconds, tokens [1, n])"""
        n = n_steps or steps
        with torch.no_grad():
            t_pre, logits = sync_time(lambda: model.prefill_static(prompt, kcs, vcs))
            first = logits.argmax(-1)

            def loop():
                tok, toks = first, [first]
                for i in range(n - 1):
                    pos_buf.fill_(T + i)
                    if graph is None:
                        logits = model.step_static(tok, pos_buf, kcs, vcs)
                    else:
                        tok_buf.copy_(tok)
                        graph[0].replay()
                        logits = graph[1]
                    tok = logits.argmax(-1)  # eager in both modes
                    toks.append(tok)
                return torch.cat(toks, dim=1)

            t_dec, toks = sync_time(loop)
        return t_pre, t_dec, toks

    def capture(finish=None):
        """Capture one decode step (after two eager warm-up steps on a side stream)."""
        with torch.no_grad():
            model.prefill_static(prompt, kcs, vcs)
            pos_buf.fill_(T)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    model.step_static(tok_buf, pos_buf, kcs, vcs)
                if finish:
                    finish()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                logits = model.step_static(tok_buf, pos_buf, kcs, vcs)
                if finish:
                    finish()
        return g, logits

    res, toks = {}, {}
    mgr_box = []  # the manager, once the model is converted

    def measure(name, graph=None):
        run_mode(graph, 4)  # warm-up
        res[name + "_prefill_s"], res[name + "_decode_s"], toks[name] = run_mode(graph)
        ahead = ""
        if mgr_box and hasattr(mgr_box[0]._be, "ahead_stats"):
            ahead = ", weights decoded ahead used / dropped so far %d / %d" % mgr_box[0]._be.ahead_stats()
        print(f"[llama8b] {name}: prefill {res[name + '_prefill_s']:.3f} s, "
              f"{(steps - 1) / res[name + '_decode_s']:.1f} tok/s{ahead}", file=sys.stderr, flush=True)

    measure("dense_eager")
    measure("dense_graph", capture())
    dense_param_bytes = sum(p.numel() * p.element_size() for p in model.parameters())

    mgr, how = make_manager(args, args.precision)
    mgr_box.append(mgr)
    t_conv, _ = sync_time(lambda: mgr.convert(model))
    torch.cuda.empty_cache()
    comp_bytes = sum(mgr.size(h) for h in mgr.meta_dict)
    comp_dense_bytes = sum(2 * int(np.prod(shp)) for shp in mgr.meta_dict.values())
    over_entropy = size_over_entropy(torch, mgr, args.precision)
    torch.cuda.empty_cache()

    # the unchanged caller: nothing but the reference's calls; Manager.linear itself sends a
    # single activation row through the fused decode-and-multiply kernel
    measure("unchanged_caller_eager")
    measure("unchanged_caller_graph", capture())
    # decompress-then-GEMM for every call, the reference's own route (bit-equal to dense)
    mgr.fused_rows = False
    mgr.decode_ahead = False
    measure("per_linear_eager")
    measure("per_linear_graph", capture())
    for ahead in ((False, True) if full else ()):
        tag = "per_block_ahead" if ahead else "per_block"
        da = neuzip_amd.DecompressAhead(mgr, model, ahead=ahead)
        with da:
            measure(tag + "_eager")
        del da
        da = neuzip_amd.DecompressAhead(mgr, model, ahead=ahead, wrap=False)
        with da:
            measure(tag + "_graph", capture(finish=da.join))
        del da
        torch.cuda.empty_cache()
    # decode fused into the matrix-vector product, Linears that share an input in one launch
    # (single-token steps only; the prefill keeps the decompress-then-GEMM path)
    mgr.fused_rows = True
    mgr.decode_ahead = True
    fused = neuzip_amd.FusedGemv(mgr, model)
    with torch.no_grad():
        model.prefill_static(prompt, kcs, vcs)
        pos_buf.fill_(T)
        fused.trace(lambda: model.step_static(tok_buf, pos_buf, kcs, vcs))
    with fused:
        measure("fused_eager")
        measure("fused_graph", capture())
    mgr._be.check()

    modes = [k[:-9] for k in res if k.endswith("_decode_s")]
    rounds_its_own_way = ("fused", "unchanged_caller")  # the fused product sums in an order of its own
    same = all(bool(torch.equal(toks["dense_eager"], toks[m])) for m in modes if not m.startswith(rounds_its_own_way))
    fused_same = bool(torch.equal(toks["fused_eager"], toks["fused_graph"]))
    fused_prefix = int((toks["fused_eager"] != toks["dense_eager"]).int().cumsum(1).eq(0).sum())
    plain_same = bool(torch.equal(toks["unchanged_caller_eager"], toks["unchanged_caller_graph"]))
    plain_prefix = int((toks["unchanged_caller_eager"] != toks["dense_eager"]).int().cumsum(1).eq(0).sum())
    comp_modes = [m for m in modes if not m.startswith("dense")]
    tok_s = {m: round((steps - 1) / res[m + "_decode_s"], 2) for m in modes}
    total = {m: res[m + "_prefill_s"] + res[m + "_decode_s"] for m in modes}
    best = max(comp_modes, key=lambda m: tok_s[m])
    best_eager = max((m for m in comp_modes if m.endswith("eager")), key=lambda m: tok_s[m])
    best_graph = max((m for m in comp_modes if m.endswith("graph")), key=lambda m: tok_s[m])
    out = {
        "metric": "llama8b_shape_compressed_decode_tok_s",
        "value": tok_s[best],
        "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": 4,
        "ms_per_step": round(res[best + "_decode_s"] / (steps - 1) * 1e3, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"Llama-3-8B-shaped random-init decoder, {layers} layers, batch 1, {T}-token "
                        f"prompt + {steps} greedy steps, Linear weights compressed (precision {args.precision})",
            "manager": how,
            "best_mode": best,
            "unchanged_caller": {
                "decode_tok_s_eager": tok_s["unchanged_caller_eager"],
                "decode_tok_s_graph": tok_s["unchanged_caller_graph"],
                "per_token_over_dense_eager": round(tok_s["dense_eager"] / tok_s["unchanged_caller_eager"], 3),
                "per_token_over_dense_graph": round(tok_s["dense_graph"] / tok_s["unchanged_caller_graph"], 3),
                "total_over_dense_eager": round(total["unchanged_caller_eager"] / total["dense_eager"], 3),
                "total_over_dense_graph": round(total["unchanged_caller_graph"] / total["dense_graph"], 3),
                "graph_tokens_equal_eager": plain_same,
                "leading_tokens_equal_to_dense": plain_prefix,
            },
            "tokens_identical_in_all_decompress_modes": same,
            "fused_graph_tokens_equal_fused_eager": fused_same,
            "fused_leading_tokens_equal_to_dense": fused_prefix,
            "fused_groups": sorted(len(g.handles) for g in fused._groups)[-4:],
            "decode_tok_s": tok_s,
            "prefill_s": {m: round(res[m + "_prefill_s"], 4) for m in modes},
            "total_s": {m: round(total[m], 4) for m in modes},
            "latency_ratio_eager": {"mode": best_eager,
                                    "total": round(total[best_eager] / total["dense_eager"], 3),
                                    "per_token": round(tok_s["dense_eager"] / tok_s[best_eager], 3)},
            "latency_ratio_graph": {"mode": best_graph,
                                    "total": round(total[best_graph] / total["dense_graph"], 3),
                                    "per_token": round(tok_s["dense_graph"] / tok_s[best_graph], 3)},
            "convert_s": round(t_conv, 3),
            "compressed_weight_bytes": comp_bytes,
            "dense_bytes_of_compressed_weights": comp_dense_bytes,
            "stored_over_dense": round(comp_bytes / comp_dense_bytes, 5),
            "exponent_bytes_over_entropy_bound": over_entropy,
            "dense_model_bytes": dense_param_bytes,
        },
    }
    del fused, mgr, model, kcs, vcs
    torch.cuda.empty_cache()
    return out


def run_llama8b(args, torch):
    print(json.dumps(llama8b_measure(args, torch, full=True)))
    return 0


def run_gpt2m(args, torch):
    print(json.dumps(gpt2m_measure(args, torch)))
    return 0


def gpt2m_measure(args, torch):
    """BASELINE config 4: GPT-2-medium-shaped model, weights kept compressed and
    re-compressed after every AdamW step; reports the codec share of the step."""
    import neuzip_amd
    from bench_models import CompressedAdamW, GPT2Shaped, ReferenceLoopSGD

    layers = args.layers or 24
    torch.manual_seed(args.seed)
    with torch.device("cuda"):
        torch.set_default_dtype(torch.bfloat16)
        model = GPT2Shaped(layers=layers, ctx=args.seq_len)
        torch.set_default_dtype(torch.float32)
    def train_step(opts):
        ids = torch.randint(0, 50257, (args.batch, args.seq_len), device="cuda")
        logits = model(ids[:, :-1])
        loss = torch.nn.functional.cross_entropy(logits.float().reshape(-1, logits.shape[-1]), ids[:, 1:].reshape(-1))
        loss.backward()
        for o in opts:
            o.step()
        return loss.detach()

    # the same model with dense bf16 weights and torch's AdamW: for scale, and (lossless
    # setting) as the loss curve the compressed run has to reproduce
    state0 = {k: v.clone() for k, v in model.state_dict().items()}
    opt = torch.optim.AdamW(model.parameters(), lr=1e-4)
    torch.manual_seed(args.seed + 1)
    dense_losses = []
    for _ in range(args.warmup):
        dense_losses.append(train_step([opt]))
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dense_losses.append(train_step([opt]))
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    dense_ms = (time.perf_counter() - t0) / args.steps * 1e3
    del opt
    # ... and with the reference's update hooks on every parameter (plain SGD inside the backward pass)
    import neuzip_amd as _nz
    from functools import partial as _partial

    class _LR:
        def get_last_lr(self):
            return [1e-4]

    dense_hooks = [p.register_post_accumulate_grad_hook(_partial(_nz.lomo_hook, _LR())) for p in model.parameters()]
    for _ in range(args.warmup):
        train_step([])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        train_step([])
    torch.cuda.synchronize()
    dense_hooks_ms = (time.perf_counter() - t0) / args.steps * 1e3
    for hd in dense_hooks:
        hd.remove()
    model.load_state_dict(state0)
    del state0
    torch.cuda.empty_cache()

    mgr, how = make_manager(args, args.precision)
    mgr.convert(model)
    comp_params = [p for p in model.parameters() if isinstance(p, neuzip_amd.nn.Parameter)]
    rest = [p for p in model.parameters() if not isinstance(p, neuzip_amd.nn.Parameter)]
    # time every codec call with events on the stream it runs on
    be = mgr._be
    spans = []
    n_calls = {"decode": 0, "encode": 0}

    depth = [0]

    def timed(fn, kind):
        def wrapper(*a, **k):
            n_calls[kind] += 1
            if depth[0]:  # inside another codec call (held writes stored by it): that one's span covers this
                return fn(*a, **k)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            depth[0] += 1
            try:
                r = fn(*a, **k)
            finally:
                depth[0] -= 1
            e1.record()
            spans.append((kind, e0, e1))
            return r
        return wrapper

    be.read, be.write = timed(be.read, "decode"), timed(be.write, "encode")
    be.read_batch = timed(be.read_batch, "decode")
    be.write_batch = timed(be.write_batch, "encode")

    def run(group, sgd_loop=False, hooks_only=False):
        """-> per-step figures with the Linears decoded one by one (group 1) or per block"""
        opt_c = ReferenceLoopSGD(comp_params, lr=1e-4) if sgd_loop else CompressedAdamW(comp_params, lr=1e-4, group=group)
        opt_d = torch.optim.AdamW(rest, lr=1e-4)

        def step():
            if hooks_only:  # the hooks registered on the parameters do all the updating
                return train_step([])
            loss = train_step([opt_c, opt_d])
            opt_d.zero_grad(set_to_none=True)
            return loss

        warm = [step() for _ in range(args.warmup)]
        torch.cuda.synchronize()
        spans.clear()
        launched = be.rewrite_stats()[0]
        t0 = time.perf_counter()
        losses = [step() for _ in range(args.steps)]
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        launched = be.rewrite_stats()[0] - launched  # every write here goes into the buffers its entry has
        dec = sum(a.elapsed_time(b) for k, a, b in spans if k == "decode") * 1e-3
        enc = sum(a.elapsed_time(b) for k, a, b in spans if k == "encode") * 1e-3
        return {
            "ms_per_step": round(wall / args.steps * 1e3, 3),
            "codec_share_of_step": round((dec + enc) / wall, 4),
            "decode_s_per_step": round(dec / args.steps, 5),
            "encode_s_per_step": round(enc / args.steps, 5),
            "decode_launches_per_step": sum(1 for k, _, _ in spans if k == "decode") / args.steps,
            "encodes_per_step": sum(1 for k, _, _ in spans if k == "encode") / args.steps,
            "encode_launches_per_step": launched / args.steps,
            "first_loss": round(float(losses[0]), 4),
            "last_loss": round(float(losses[-1]), 4),
        }, wall, warm + losses

    # per block first: it starts from the very weights, data and optimizer state the dense run
    # started from, so with a lossless manager its losses must be the dense run's, bit for bit
    per_block_linears = len(comp_params) // max(1, layers)
    torch.manual_seed(args.seed + 1)
    da = neuzip_amd.DecompressAhead(mgr, model, ahead=False)  # small blocks share a launch (up to 16 tensors)
    per_launch = max(da.tensors_per_launch)
    with da:
        per_block, wall, comp_losses = run(per_launch)
    del da
    same = sum(1 for a, b in zip(dense_losses, comp_losses) if torch.equal(a, b))
    per_block["steps_with_the_dense_runs_loss"] = f"{same} of {len(dense_losses)}"
    per_block["dense_first_loss"] = round(float(dense_losses[args.warmup]), 4)
    per_block["dense_last_loss"] = round(float(dense_losses[-1]), 4)
    mgr.decode_ahead = False  # the reference's granularity: every request decodes its own tensor,
    mgr.write_behind = False  # every write is an encode launch of its own
    per_linear, _, _ = run(1)
    # the same loop, nothing but the reference's calls, with the manager's default: a request
    # decodes the weights it has learned to expect next in the same launch, and small writes
    # wait (as copies) until 16 of them share a launch
    mgr.decode_ahead = True
    mgr.write_behind = True
    per_linear_learned, _, _ = run(1)
    hits, waste = mgr._be.ahead_stats()
    per_linear_learned["weights_decoded_ahead_used"] = hits
    per_linear_learned["weights_decoded_ahead_dropped"] = waste
    # the reference's own update statement (plain SGD through read and write, train_clm.py:822-833)
    # in place of AdamW: first at the reference's granularity, then with the manager's defaults
    mgr.decode_ahead = mgr.write_behind = False
    sgd_loop_plain, _, _ = run(1, sgd_loop=True)
    mgr.decode_ahead = mgr.write_behind = True
    sgd_loop, _, _ = run(1, sgd_loop=True)

    # the reference's update hooks (neuzip/__init__.py:16-35): every parameter is updated, and a
    # compressed one written back, from a post-accumulate-grad hook in the middle of the backward pass
    class _FixedLR:
        def get_last_lr(self):
            return [1e-4]

    from functools import partial

    def with_hooks(params_and_hooks):
        return [p.register_post_accumulate_grad_hook(partial(h, _FixedLR())) for p, h in params_and_hooks]

    hooked = [(p, neuzip_amd.compressed_lomo_hook) for p in comp_params] + [(p, neuzip_amd.lomo_hook) for p in rest]
    mgr.decode_ahead = mgr.write_behind = False
    handles = with_hooks(hooked)
    lomo_plain, _, _ = run(1, hooks_only=True)
    mgr.decode_ahead = mgr.write_behind = True
    lomo, _, _ = run(1, hooks_only=True)
    for hd in handles:
        hd.remove()
    mgr._be.check()
    # writes that went into the entries' existing buffers (no allocation, no wait for the size)
    in_place, outgrown = be.rewrite_stats()
    rewrites = {"write_batches_in_place": in_place, "entries_that_outgrew_their_buffer": outgrown,
                "write_calls": n_calls["encode"]}
    n_comp = len(comp_params)
    stored_ratio = round(sum(mgr.size(p._handle) for p in comp_params) /
                         sum(2 * int(np.prod(p._shape)) for p in comp_params), 5)
    over_entropy = size_over_entropy(torch, mgr, args.precision, [p._handle for p in comp_params])  # the weights as trained
    del mgr, model, comp_params, rest
    torch.cuda.empty_cache()

    # Which part of a loss difference, if there is one, belongs to the codec: a dense model and
    # its converted twin trained side by side on the same data, the dense gradients handed to
    # both optimizers, every decoded weight compared with the dense weight after every step
    # (bench_models.lockstep_adamw).  The losses above compare two separate runs and so also
    # see whatever the GEMM and attention kernels do differently from run to run.
    lockstep = None
    if args.verify_steps > 0:
        from bench_models import lockstep_adamw

        def twin():
            torch.manual_seed(args.seed)
            with torch.device("cuda"):
                torch.set_default_dtype(torch.bfloat16)
                try:
                    return GPT2Shaped(layers=layers, ctx=args.seq_len)
                finally:
                    torch.set_default_dtype(torch.float32)

        dense_twin, comp_twin = twin(), twin()
        mgr2, _ = make_manager(args, 7)
        mgr2.convert(comp_twin)
        g = torch.Generator(device="cuda").manual_seed(args.seed + 2)
        da2 = neuzip_amd.DecompressAhead(mgr2, comp_twin, ahead=False)
        with da2:
            lockstep = lockstep_adamw(
                dense_twin, comp_twin, mgr2,
                lambda i: torch.randint(0, 50257, (args.batch, args.seq_len), device="cuda", generator=g),
                steps=args.verify_steps, group=max(da2.tensors_per_launch))
        del da2
        mgr2._be.check()
    tokens = args.batch * (args.seq_len - 1) * args.steps
    out = {
        "metric": "gpt2m_shape_compressed_training_tok_s",
        "value": round(tokens / wall, 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": per_block["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"GPT-2-medium-shaped random-init model, {layers} layers, batch {args.batch} x seq {args.seq_len}, "
                        f"bf16 weights compressed (precision {args.precision}), re-compressed after each AdamW step",
            "dense_bf16_torch_adamw_ms_per_step": round(dense_ms, 3),
            "dense_bf16_update_hooks_ms_per_step": round(dense_hooks_ms, 3),
            "tensors_per_decode_and_write_launch": per_launch,
            "decode_per_block": per_block,
            "decode_per_linear": per_linear,
            "decode_per_linear_order_learned": per_linear_learned,
            "reference_sgd_loop_per_linear": sgd_loop_plain,
            "reference_sgd_loop_order_learned": sgd_loop,
            "reference_update_hooks_per_linear": lomo_plain,
            "reference_update_hooks_order_learned": lomo,
            "lockstep_check_lossless": lockstep,
            "rewrites": rewrites,
            "compressed_tensors": n_comp,
            "manager": how,
            "stored_over_dense": stored_ratio,
            "exponent_bytes_over_entropy_bound": over_entropy,
        },
    }
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU codec path; this build runs on one GPU only "
              "(--gpus must be 1).", file=sys.stderr)
        return 2

    import torch

    from neuzip_amd import _lib as lib_mod

    L = lib_mod.load()  # raises if the HIP extension is missing: there is no fallback
    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        return 2

    if args.lane_symbols is None:  # model workloads: tensors of many sizes, geometry per tensor
        args.lane_symbols = 0 if args.workload == "tensor" else -1

    if args.calibrate_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "5 device copies", "bytes_read_per_copy": 256 << 20,
                          "bytes_written_per_copy": 256 << 20}))
        return 0

    if args.protocol_probe:
        return protocol_probe(args, torch, L, lib_mod)
    if args.encode_phases:
        return encode_phases(args, torch, L, lib_mod)
    if args.workload == "llama8b":
        return run_llama8b(args, torch)
    if args.workload == "gpt2m":
        return run_gpt2m(args, torch)

    n = args.rows * args.cols
    chunk = args.chunk_size or lib_mod.DEFAULT_CHUNK
    lane = args.lane_symbols or (lib_mod.DEFAULT_LANE_SYMS if chunk == lib_mod.DEFAULT_CHUNK else
                                 344 if chunk == 65536 else max(16, chunk // 512))
    R = max(1, args.rotate)
    dense_bytes = 2 * n
    ws = Workspace(torch, L, lib_mod, max(n, STRESS_ROWS * STRESS_COLS if not args.no_stress else n), chunk, lane)

    # ---- R independent copies of the workload (seeds seed .. seed+R-1), each with its own
    # compressed streams and its own output: a rotation over them touches R x (C + P + 2N)
    # bytes between two uses of the same bytes, far more than the 256 MB last-level cache
    denses = [normal_weight(torch, args.rows, args.cols, args.seed + i) for i in range(R)]
    outs = [torch.empty_like(d) for d in denses]
    sets = [ws.encode(d, args.precision) for d in denses]
    for st, o in zip(sets, outs):
        ws.decode(st, o, check=True)
    torch.cuda.synchronize()

    # ---- parity of this very run against the oracle-independent closed form, every set
    bit_exact = all(bool(torch.equal(o.view(torch.int16), closed_form_torch(torch, d, args.precision)))
                    for d, o in zip(denses, outs))
    headline_out = outs[0].view(torch.int16).cpu().numpy().view(np.uint16).copy()
    host_bits = denses[0].view(torch.int16).cpu().numpy().view(np.uint16)

    # ---- the timed region.  A step is one pass over the batch of R stored weights (R launches).
    # The GPU's clocks take several milliseconds of load to settle (the first ~100 launches after
    # an idle period run up to 10 % slower), so `settle` untimed launches precede the W warm-up
    # steps; their number is reported.
    def rotation():
        for st, o in zip(sets, outs):
            ws.decode(st, o)

    settle = 0
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_s:
        rotation()
        torch.cuda.synchronize()
        settle += R
    wall, step_time = time_launches(torch, rotation, args.steps, args.warmup)
    ms_per_step = wall / args.steps * 1e3
    value = R * dense_bytes * args.steps / wall / 1e9
    algo_bytes = sum(st.total + st.packed_bytes + dense_bytes for st in sets) / R  # C + P + 2N, mean over the sets
    cold_launch = step_time / R
    cold = roofline_block(algo_bytes, cold_launch, args.precision,
                          working_set=int(R * algo_bytes), launches=args.steps * R,
                          note=f"rotation over {R} independent (container, packed, output) sets: out of the "
                               "last-level cache; default output policy (ordinary stores up to 128 MiB)")
    cold["traffic"], cold["traffic_source"] = recorded_traffic(
        f"nz_decode_kernel<{args.precision}>, {args.rows}x{args.cols}, chunk {chunk}, lane {lane}, rotating {R} sets")

    # Two more views of the same cold inputs.  (1) The output goes to ONE buffer that every
    # decode reuses, as in the library's read path (the weight is consumed by the GEMM that
    # follows and the allocator or the per-block slot hands the same memory to the next
    # decode): only compressed bytes come from HBM, the output lines are already cached.
    # (2) Everything rotates as in the headline, but the output is written with streaming
    # stores (NZ_DECODE_STREAM_OUT, the default only for tensors above 128 MiB): faster for
    # a decode whose output nobody reads soon, slower for decode + GEMM.
    extra = {}
    if R > 1 and not args.no_hot:
        def rotation_one_out():
            for st in sets:
                ws.decode(st, outs[0])

        def rotation_streaming():
            for st, o in zip(sets, outs):
                ws.decode(st, o, flags=lib_mod.DECODE_STREAM_OUT)

        for name, fn, note in (
                ("roofline_cold_reused_output", rotation_one_out,
                 f"{R} stored tensors in rotation, decoded into one reused output buffer"),
                ("roofline_cold_streaming_stores", rotation_streaming,
                 f"rotation over {R} independent stored tensors and outputs, streaming stores forced")):
            _, t_step = time_launches(torch, fn, args.steps, args.warmup)
            extra[name] = roofline_block(algo_bytes, t_step / R, args.precision, working_set=int(R * algo_bytes),
                                         launches=args.steps * R, note=note)

    # the same kernel on ONE stored tensor over and over (what a single hot layer sees): its
    # 223 MB working set stays in the 256 MB last-level cache, so this is not an HBM figure
    hot = None
    if R > 1 and not args.no_hot:
        _, hot_launch = time_launches(torch, lambda: ws.decode(sets[0], outs[0]), args.steps * R, args.warmup * R)
        a0 = sets[0].total + sets[0].packed_bytes + dense_bytes
        hot = roofline_block(a0, hot_launch, args.precision, working_set=a0, launches=args.steps * R,
                             note="one stored tensor decoded repeatedly: resident in the 256 MB last-level cache")
        hot["traffic"], hot["traffic_source"] = None, None

    # entropy bound of the exponent stream (order 0, per 64 KiB chunk), set 0
    a = host_bits.astype(np.uint32)
    if args.precision == 7:
        exps_host = ((a >> 7) & 0xFF).astype(np.uint8)
    else:
        s = args.precision
        exps_host = ((((a & 0x7FFF) + (1 << (6 - s))) & 0x7FFF) >> 7).astype(np.uint8)
    bound = 0.0
    for c in range(0, n, 65536):
        cnt = np.bincount(exps_host[c:c + 65536], minlength=256).astype(np.float64)
        nz = cnt[cnt > 0]
        bound += -(nz * np.log2(nz / nz.sum())).sum() / 8.0
    packed_ref_bytes = int(L.nz_packed_bytes(n, args.precision))

    result = {
        "metric": "bf16_decompress_GBps",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u16",
        "data": "synthetic",
        "config": {
            "workload": f"batch of {R} lossless-compressed bf16 weights {args.rows}x{args.cols} N(0,0.02), seeds "
                        f"{args.seed}..{args.seed + R - 1}: fused rANS decode + merge, precision {args.precision}; "
                        f"one step decodes the batch once ({R} launches)",
            "elements_per_weight": n,
            "weights_per_step": R,
            "precision": args.precision,
            "chunk_size": chunk,
            "lane_symbols": lane,
            "bit_exact": bit_exact,
            "settle_launches_before_warmup": settle,
            "compressed_exponent_bytes": sets[0].total,
            "packed_sign_mantissa_bytes": sets[0].packed_bytes,
            "stored_over_dense": round((sets[0].total + sets[0].packed_bytes) / dense_bytes, 5),
            "exponent_bytes_over_entropy_bound": round((sets[0].total + sets[0].packed_bytes - packed_ref_bytes) / bound, 5),
        },
        "roofline": cold,
        "roofline_cold": cold,
    }
    result.update(extra)
    if hot is not None:
        result["roofline_hot"] = hot

    # ---- BASELINE config 5: the 8192 x 28672 stress tensor (448 MiB dense: out of cache by itself) ----
    if not args.no_stress:
        stress = stress_weight(torch, STRESS_ROWS, STRESS_COLS, args.seed)
        s_out = torch.empty_like(stress)
        cfg5 = {"workload": f"{STRESS_ROWS}x{STRESS_COLS} bf16, Student-t(3) x 0.02, 1 % zeros, 0.1 % subnormals, "
                            "16 outlier columns x 50"}
        k5 = max(100, args.steps)
        for s in (7, 3):
            st = ws.encode(stress, s)
            ws.decode(st, s_out, check=True)
            ok = bool(torch.equal(s_out.view(torch.int16), closed_form_torch(torch, stress, s)))
            _, m_d, _ = settled_launches(torch, lambda: ws.decode(st, s_out), k5, 3, args.settle_s / 2)
            _, m_e, _ = settled_launches(torch, lambda: ws.encode_into(stress, s, st), k5, 2, args.settle_s / 2)
            ab = st.total + st.packed_bytes + 2 * stress.numel()
            cfg5[f"precision_{s}"] = {
                "bit_exact": ok,
                "decode": roofline_block(ab, m_d, s, working_set=ab, launches=k5),
                "encode_GBps": round(2 * stress.numel() / m_e / 1e9, 1),
                "encode_hbm_frac": round(ab / m_e / 1e9 / HBM_PEAK_GBPS, 4),
                "stored_over_dense": round((st.total + st.packed_bytes) / (2 * stress.numel()), 5),
            }
            del st
        result["stress_8192x28672"] = cfg5
        del stress, s_out
        torch.cuda.empty_cache()

    # ---- encode throughput and the precision sweep (reported, not `value`); rotating like the headline.
    # Every point gets the headline's protocol: its own settle phase of the very launches it times
    # (a point that starts right after allocations, host-synchronised encodes or another kernel
    # otherwise runs its first launches at clocks that are still moving) and 100 launches or more
    # between the two events; wall time over event time of the timed region is reported beside it.
    if not args.no_sweep:
        sweep = {}
        k = max(-(-100 // R), args.steps // 2)
        for s in (7, 3, 1, 0):
            ss = sets if s == args.precision else [ws.encode(d, s) for d in denses]

            def dec():
                for st, o in zip(ss, outs):
                    ws.decode(st, o)

            def enc():
                for d, st in zip(denses, ss):
                    ws.encode_into(d, s, st)

            w_d, m_d, u_d = settled_launches(torch, dec, k, 2, args.settle_s / 2)
            w_e, m_e, u_e = settled_launches(torch, enc, k, 2, args.settle_s / 2)
            ab = sum(st.total + st.packed_bytes + dense_bytes for st in ss) / R
            sweep[str(s)] = {
                "decode_GBps": round(dense_bytes / (m_d / R) / 1e9, 1),
                "decode_hbm_frac": round(ab / (m_d / R) / 1e9 / HBM_PEAK_GBPS, 4),
                "decode_launch_us": round(m_d / R * 1e6, 2),
                "decode_wall_over_event": round(w_d / (m_d * k), 3),
                "encode_GBps": round(dense_bytes / (m_e / R) / 1e9, 1),
                "encode_hbm_frac": round(ab / (m_e / R) / 1e9 / HBM_PEAK_GBPS, 4),
                "encode_launch_us": round(m_e / R * 1e6, 2),
                "encode_wall_over_event": round(w_e / (m_e * k), 3),
                "launches_timed": k * R,
                "untimed_launches_before": [u_d * R, u_e * R],
                "stored_over_dense": round((ss[0].total + ss[0].packed_bytes) / dense_bytes, 5),
            }
            if ss is not sets:
                del ss
        result["sweep"] = sweep

    # ---- CPU baseline: the oracle (same container format) on the host cores ----
    if not args.no_cpu_baseline:
        from oracle import oracle as O

        O.build()
        threads = args.cpu_threads or len(os.sched_getaffinity(0))
        comp_h = sets[0].comp[: sets[0].total].cpu().numpy()
        packed_h = sets[0].packed[: sets[0].packed_bytes].cpu().numpy()
        times = []
        t_budget = time.perf_counter()
        for _ in range(5):
            t0 = time.perf_counter()
            rc, rec = O.decompress_bf16(comp_h, packed_h, n, args.precision, threads=threads)
            times.append(time.perf_counter() - t0)
            if rc != 0:
                raise RuntimeError("oracle failed to decode the GPU container")
            if time.perf_counter() - t_budget > 30:
                break
        cpu_ok = bool(np.array_equal(rec, headline_out))
        result["cpu_baseline"] = {
            "value": round(dense_bytes / statistics.median(times) / 1e9, 3),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"one {args.rows}x{args.cols} weight of the batch decoded {len(times)} times by the C oracle "
                      f"({threads} threads over chunks), median",
            "matches_gpu_output": cpu_ok,
        }

    del sets, denses, outs, ws
    torch.cuda.empty_cache()

    # ---- the second half of the metric: tokens/s of an 8B-shaped compressed decoder ----
    if not args.no_llama:
        import copy

        largs = copy.copy(args)
        largs.precision, largs.lane_symbols = 7, -1
        try:
            lm = llama8b_measure(largs, torch, full=False)
            cfg = lm["config"]
            result["llama8b_shape"] = {
                "workload": cfg["workload"],
                "manager": cfg["manager"],
                "unchanged_caller": cfg["unchanged_caller"],
                "decode_tok_s": cfg["decode_tok_s"],
                "latency_ratio_eager": cfg["latency_ratio_eager"],
                "latency_ratio_graph": cfg["latency_ratio_graph"],
                "tokens_identical_in_all_decompress_modes": cfg["tokens_identical_in_all_decompress_modes"],
                "fused_graph_tokens_equal_fused_eager": cfg["fused_graph_tokens_equal_fused_eager"],
                "stored_over_dense": cfg["stored_over_dense"],
                "exponent_bytes_over_entropy_bound": cfg["exponent_bytes_over_entropy_bound"],
            }
        except Exception as e:  # the codec line above stands on its own
            result["llama8b_shape"] = {"error": f"{type(e).__name__}: {e}"}
        torch.cuda.empty_cache()

    # ---- BASELINE config 4: a GPT-2-medium-shaped model trained with its weights kept compressed ----
    if not args.no_gpt2m:
        import copy

        gargs = copy.copy(args)
        gargs.precision, gargs.lane_symbols, gargs.chunk_size = 7, -1, 0
        gargs.steps, gargs.warmup, gargs.verify_steps = 20, 3, 5
        try:
            gm = gpt2m_measure(gargs, torch)
            cfg = gm["config"]
            pb = cfg["decode_per_block"]
            result["gpt2m_shape"] = {
                "workload": cfg["workload"],
                "manager": cfg["manager"],
                "timed_steps": gargs.steps,
                "tensors_per_decode_and_write_launch": cfg["tensors_per_decode_and_write_launch"],
                "tokens_per_s": gm["value"],
                "ms_per_step_dense_bf16_adamw": cfg["dense_bf16_torch_adamw_ms_per_step"],
                "ms_per_step_dense_bf16_update_hooks": cfg["dense_bf16_update_hooks_ms_per_step"],
                "ms_per_step_compressed_decode_per_block": pb["ms_per_step"],
                "ms_per_step_compressed_decode_per_linear": cfg["decode_per_linear"]["ms_per_step"],
                "ms_per_step_compressed_unchanged_caller": cfg["decode_per_linear_order_learned"]["ms_per_step"],
                "ms_per_step_reference_sgd_loop": cfg["reference_sgd_loop_order_learned"]["ms_per_step"],
                "ms_per_step_reference_sgd_loop_per_linear": cfg["reference_sgd_loop_per_linear"]["ms_per_step"],
                "ms_per_step_reference_update_hooks": cfg["reference_update_hooks_order_learned"]["ms_per_step"],
                "ms_per_step_reference_update_hooks_per_linear": cfg["reference_update_hooks_per_linear"]["ms_per_step"],
                "codec_share_of_step_per_block": pb["codec_share_of_step"],
                "codec_share_of_step_per_linear": cfg["decode_per_linear"]["codec_share_of_step"],
                "codec_share_of_step_unchanged_caller": cfg["decode_per_linear_order_learned"]["codec_share_of_step"],
                "steps_with_the_dense_runs_loss": pb["steps_with_the_dense_runs_loss"],
                "rewrites": cfg["rewrites"],
                "lockstep_check_lossless": cfg["lockstep_check_lossless"],
                "stored_over_dense": cfg["stored_over_dense"],
                "exponent_bytes_over_entropy_bound": cfg["exponent_bytes_over_entropy_bound"],
            }
        except Exception as e:
            result["gpt2m_shape"] = {"error": f"{type(e).__name__}: {e}"}

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
