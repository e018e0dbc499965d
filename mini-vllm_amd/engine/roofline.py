"""Prices the kernels of a profiled step: which kernel ran how long, how many bytes it had to
move, how many floating-point operations it did, and what share of the machine's peaks that is.

Two sources are joined. The *ledger* is written by the kernel front end (``Ops.ledger``) while a
step runs or is recorded into a graph: one line per launch with the entry point, the bytes the
launch has to read and write and its operations, in launch order. The *trace* is the
``*_kernel_trace.csv`` that ``rocprofv3 --kernel-trace --output-format csv`` writes: every kernel
dispatch of a whole run with its name and its start and end time. The stream of a step is in launch
order, so the ledger of one step, turned into the kernel names each entry point launches, is a
pattern that occurs in the trace once for every time such a step ran. Every occurrence is found,
and each launch is priced with its median time over the occurrences.
"""
from __future__ import annotations

import csv
import re
import statistics
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

PEAK_HBM_BYTES = 8.0e12
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

_LIBRARY = r"^((Custom_)?Cijk_|void hipblaslt|hipblaslt|.*rocblaslt)"
# entry point -> (the kernel a call starts with, the kernel that may follow it within the same call, the
# most kernels one call launches)
KERNELS_OF: Dict[str, Tuple[str, Optional[str], int]] = {
    "mv_embedding": (r"\bembedding(_gather)?_kernel", None, 1),
    "mv_add_rmsnorm": (r"\badd_rmsnorm(_vec)?_kernel", None, 1),
    "mv_add_rmsnorm_split": (r"\badd_rmsnorm(_vec)?_kernel", None, 1),
    "mv_rmsnorm": (r"\brmsnorm_kernel", None, 1),
    "mv_qk_norm_rope_store": (r"\b(qk_norm_rope_store(_vec)?_kernel|qkv_prompt_vec_kernel)", r"\bstore_v_pages_kernel", 2),
    "mv_swiglu": (r"\bswiglu(_vec)?_kernel", None, 1),
    "mv_gemm_skinny": (r"\bgemm_skinny_kernel", None, 1),
    "mv_gemm_skinny_norm": (r"\bgemm_skinny_kernel", None, 1),
    "mv_gemm_skinny_swiglu": (r"\bgemm_skinny_kernel", None, 1),
    "mv_gemm_skinny_fold": (r"\bgemm_skinny_kernel", None, 1),
    "mv_gemm_skinny_scaled": (r"\bgemm_skinny_kernel", None, 1),
    "mv_scale_rows": (r"\bscale_rows_kernel", None, 1),
    "mv_gemm_ref": (r"\bgemm_nt_kernel", None, 1),
    "mv_gemm_mid": (r"\bgemm_mid_kernel", r"\bgemm_mid_reduce_kernel", 2),
    "mv_gemm_tile": (r"\bgemm_tile_kernel", r"\bgemm_mid_reduce_kernel", 2),
    "mv_gemm_lt": (_LIBRARY, _LIBRARY, 3),
    "mv_attention_ref": (r"\battention_ref_kernel", None, 1),
    "mv_attention_decode": (r"\battention_decode(_wave)?_kernel", r"\battention_merge(_range)?_kernel", 2),
    "mv_attention_decode_fused": (r"\battention_decode(_wave)?_kernel", r"\battention_merge(_range)?_kernel", 2),
    "mv_attention_prefill": (r"\battention_prefill_kernel", None, 1),
    "mv_sample": (r"\bsample(_partial)?_kernel", r"\bsample_kernel", 2),
}
_OURS = re.compile("|".join(f"(?:{p})" for spec in KERNELS_OF.values() for p in spec[:2] if p))


@dataclass
class Launch:
    """One line of the ledger. ``per_key_bytes`` and ``per_pair_flops`` are the parts of an
    attention launch that grow with the context: bytes per key in the cache of the step's sequences
    and operations per (query, visible key) pair, so that a step recorded at one context length can
    be priced at the mean length of the profiled steps."""
    entry: str
    bytes: int
    flops: int
    keys: int = 0
    pairs: int = 0
    per_key_bytes: int = 0
    per_pair_flops: int = 0

    def priced(self, keys: Optional[int] = None, pairs: Optional[int] = None) -> Tuple[int, int]:
        k = self.keys if keys is None else keys
        p = self.pairs if pairs is None else pairs
        return self.bytes + k * self.per_key_bytes, self.flops + p * self.per_pair_flops


def launches(ledger: Sequence[tuple]) -> List[Launch]:
    """The front end's ledger lines (plain tuples, short ones for launches without a context part)."""
    return [Launch(*line) for line in ledger]


def one_step(ledger: Sequence[Launch]) -> List[Launch]:
    """The launches of the first model step in a ledger that holds several in a row (a graph of
    repeated decode steps): from the first embedding up to the next."""
    starts = [i for i, l in enumerate(ledger) if l.entry == "mv_embedding"]
    if not starts:
        return list(ledger)
    end = starts[1] if len(starts) > 1 else len(ledger)
    return list(ledger[starts[0]:end])


def read_trace(path: str) -> List[Tuple[str, float]]:
    """(kernel name, microseconds) of every dispatch, in start order."""
    rows = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            if "Kernel_Name" not in r or "Start_Timestamp" not in r:
                raise ValueError(f"{path} is not a rocprofv3 kernel trace (columns Kernel_Name, Start_Timestamp, "
                                 f"End_Timestamp are needed; the *_kernel_trace.csv file has them)")
            rows.append((int(r["Start_Timestamp"]), r["Kernel_Name"], (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3))
    rows.sort()
    return [(n, d) for _, n, d in rows]


def short_name(kernel: str) -> str:
    name = kernel[5:] if kernel.startswith("void ") else kernel
    depth, out = 0, []
    for ch in name:                                # cut the parameter list, keep template arguments
        if ch == "(" and depth == 0:
            break
        depth += ch == "<"
        depth -= ch == ">"
        out.append(ch)
    name = "".join(out).replace("__hip_bfloat16", "bf16").replace(", ", ",")
    if name.startswith(("Cijk_", "Custom_Cijk_")):
        name = name[name.index("Cijk_"):]
        m = re.search(r"MT(\d+x\d+x\d+)", name)
        kind = name.split("_")[3] if name.count("_") > 3 else ""
        name = f"hipBLASLt {kind} MT{m.group(1)}" if m else name[:40]
    return name[:64]


@dataclass
class Window:
    times: List[List[float]]                       # per ledger line: the time of each kernel it launched
    names: List[List[str]]
    other: float                                   # kernels of other libraries between them (torch's fills and copies)
    other_count: int


def _align(trace: Sequence[Tuple[str, float]], start: int, patterns, limits) -> Optional[Tuple[Window, int]]:
    """``patterns``: per ledger line the kernel a launch starts with and the one that may follow it
    (two products of the same kernel in a row are two launches, not one launch's pair)."""
    i, n = start, len(trace)
    times, names, other, other_count = [], [], 0.0, 0
    for (pat, follow), limit in zip(patterns, limits):
        while i < n and not _OURS.search(trace[i][0]):
            other += trace[i][1]
            other_count += 1
            i += 1
        got_t, got_n = [], []
        while i < n and len(got_t) < limit and (pat if not got_t else follow) is not None \
                and (pat if not got_t else follow).search(trace[i][0]):
            got_t.append(trace[i][1])
            got_n.append(trace[i][0])
            i += 1
        if not got_t:
            return None
        times.append(got_t)
        names.append(got_n)
    return Window(times, names, other, other_count), i


def find_windows(trace: Sequence[Tuple[str, float]], ledger: Sequence[Launch], most: int = 256) -> List[Window]:
    """Every place in the trace where the kernels of ``ledger`` follow each other, the last first."""
    patterns = [(re.compile(KERNELS_OF[l.entry][0]), re.compile(KERNELS_OF[l.entry][1]) if KERNELS_OF[l.entry][1] else None)
                for l in ledger]
    limits = [KERNELS_OF[l.entry][2] for l in ledger]
    first = patterns[0][0]
    windows, taken_from = [], len(trace)
    for start in range(len(trace) - 1, -1, -1):
        if not first.search(trace[start][0]):
            continue
        hit = _align(trace, start, patterns, limits)
        if hit is None or hit[1] > taken_from:
            continue
        windows.append(hit[0])
        taken_from = start
        if len(windows) >= most:
            break
    return windows


@dataclass
class Row:
    kernel: str
    calls: int = 0
    us: float = 0.0                                # all calls of a step together
    bytes: int = 0
    flops: int = 0
    entries: set = field(default_factory=set)


def kernel_table(trace_path: str, ledger: Sequence[Launch], dtype: str, keys: Optional[int] = None,
                 pairs: Optional[int] = None, title: str = "", wall_ms: Optional[float] = None) -> str:
    """The table as text. Launches of one kernel with the same bytes and operations share a row. A
    launch that makes two kernels (keys split over workgroups and merged, partial sums and their
    reduction) is priced as a whole on the row of its first kernel, the second kernel's time beside
    it, since the bytes between the two are part of what the pair has to move."""
    trace = read_trace(trace_path)
    found = find_windows(trace, ledger)
    # steps of another batch size launch the same entry points with other kernels (template
    # arguments differ): the occurrences are sorted by the exact kernels they hold and the largest
    # group is kept, so the trace should come from a run that is mostly this kind of step
    groups: Dict[Tuple, List[Window]] = {}
    for w in found:
        groups.setdefault(tuple(n for names in w.names for n in names), []).append(w)
    windows = max(groups.values(), key=len) if groups else []
    if not windows:
        seen = sorted({short_name(n) for n, _ in trace if _OURS.search(n)})
        raise ValueError(f"the trace {trace_path} holds no run of the {len(ledger)} launches of this step "
                         f"(first {ledger[0].entry}); kernels of this engine in it: {', '.join(seen) or 'none'}")
    rows: Dict[Tuple, Row] = {}
    order: List[Tuple] = []
    for j, launch in enumerate(ledger):
        samples = [sum(w.times[j]) for w in windows]
        us = statistics.median(samples)
        b, fl = launch.priced(keys, pairs)
        kernel = " + ".join(dict.fromkeys(short_name(n) for n in windows[0].names[j]))
        key = (kernel, b, fl)
        if key not in rows:
            rows[key] = Row(kernel)
            order.append(key)
        r = rows[key]
        r.calls += 1
        r.us += us
        r.bytes += b
        r.flops += fl
        r.entries.add(launch.entry)
    total_us = sum(r.us for r in rows.values())
    other_us = statistics.median(w.other for w in windows)
    other_n = int(statistics.median(w.other_count for w in windows))
    peak_f = PEAK_FLOPS[dtype]
    lines = []
    if title:
        lines.append(title)
    lines.append(f"{len(windows)} occurrences of the step in the trace ({len(found) - len(windows)} more with other kernels left out); "
                 f"times are medians; peaks: HBM 8 TB/s, "
                 f"{dtype} {peak_f / 1e12:.1f} TFLOP/s")
    head = f"{'kernel':64s} {'calls':>5s} {'us/call':>8s} {'us/step':>8s} {'%step':>6s} {'KB/call':>9s} {'GB/s':>7s} {'%HBM':>6s} {'MFLOP/call':>10s} {'TFLOP/s':>8s} {'%peak':>6s}"
    lines.append(head)
    lines.append("-" * len(head))
    for key in sorted(order, key=lambda k: -rows[k].us):
        r = rows[key]
        per = r.us / r.calls
        gbs = r.bytes / r.calls / (per * 1e-6) / 1e9 if per > 0 else 0.0
        tfl = r.flops / r.calls / (per * 1e-6) / 1e12 if per > 0 else 0.0
        lines.append(f"{r.kernel:64s} {r.calls:5d} {per:8.2f} {r.us:8.1f} {100 * r.us / total_us:6.1f} "
                     f"{r.bytes / r.calls / 1e3:9.1f} {gbs:7.0f} {100 * gbs * 1e9 / PEAK_HBM_BYTES:6.1f} "
                     f"{r.flops / r.calls / 1e6:10.2f} {tfl:8.2f} {100 * tfl * 1e12 / peak_f:6.2f}")
    lines.append("-" * len(head))
    all_bytes = sum(r.bytes for r in rows.values())
    all_flops = sum(r.flops for r in rows.values())
    n_launch = sum(len(t) for t in windows[0].times)
    lines.append(f"{'all kernels of the step (' + str(n_launch) + ' launches)':64s} {'':5s} {'':8s} {total_us:8.1f} {100.0:6.1f} "
                 f"{all_bytes / 1e3:9.0f} {all_bytes / (total_us * 1e-6) / 1e9:7.0f} "
                 f"{100 * all_bytes / (total_us * 1e-6) / PEAK_HBM_BYTES:6.1f} {all_flops / 1e6:10.0f} "
                 f"{all_flops / (total_us * 1e-6) / 1e12:8.2f} {100 * all_flops / (total_us * 1e-6) / peak_f:6.2f}")
    if other_n:
        lines.append(f"kernels of other libraries inside the step (fills, copies): {other_n} launches, {other_us:.1f} us")
    if wall_ms is not None:
        lines.append(f"the step on the clock: {wall_ms * 1e3:.1f} us; not inside a kernel: {wall_ms * 1e3 - total_us - other_us:.1f} us "
                     f"({n_launch + other_n} launches in a row)")
    return "\n".join(lines)
