"""Benchmark of the multi-adapter LoRA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config {all,1,2,3,4,5,mid,5dec}] [--layers L]

A step is one pass of one synthetic batch through the LoRA computation of `layers` decoder
layers (every projection of the configuration), issued through the reference-shaped API and
replayed as one HIP graph, with all inputs resident in HBM.

With no --config the run measures the five benchmark configurations one after the other (and, under
"extra", one mid-size prefill batch and the decode tokens of configuration 5 on their own as a decode
batch) and prints ONE JSON line.  Its top level is the BGMV decode configuration
(cfg2: 256 bf16 tokens over 128 resident rank-8 adapters, 5 % of the tokens without adapter, LoRA
on q/k/v/o): metric/value = tokens x layers per second of the whole step over exactly K steps.
"configs" holds the same figures for every configuration; "roofline_min" the lowest HBM-roofline
fraction of any kernel kind in configurations 1-4.

Per configuration: "ms_per_step" is the median of several timing windows of K steps.  "kernels" holds, per
kernel kind: "n" launches per layer, "MB" algorithmic HBM bytes per launch (10^6 bytes), "us" the average launch
duration in a graph that holds only that kind, "in_step_us" its duration inside the whole step - (replay time of
the whole-step graph - replay time of the same graph without that kind) / launches, so a kernel that runs slower
behind another kind's dirty cache lines is charged for it - and "frac" = MB / in_step_us / 8 TB/s.  All replay
times come from events recorded on the stream the graphs are launched on.  "roofline" repeats the kind that takes
most of the step (achieved = MB / in_step_us); "traffic" is the HBM-side bytes per launch from the counter passes
kept in profiles/traffic.json (not from this run).  "cpu_baseline" = the oracle's restatement of the reference's
per-adapter masked matmul loop timed on the host cores on one layer of the same batch.
"ceiling" is what plain torch operations reach in the same process, as graph nodes timed the same way: a
device-to-device copy of 1 GiB (bytes read + bytes written per second), a copy that moves 32 MiB (16 MiB each
way, buffers rotated through 512 MiB), and a one-element kernel (the cost of a graph node).
"""

import argparse
import json
import os
import statistics
import sys
import time
from collections import defaultdict

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--config", default="all", choices=["all", "1", "2", "3", "4", "5", "mid", "5dec", "2stk"])
    p.add_argument("--windows", type=int, default=5, help="timing windows of --steps steps per configuration")
    p.add_argument("--cpu-budget", type=float, default=0.0,
                   help="seconds of host time for the CPU baseline of one configuration (0 = the default share)")
    p.add_argument("--layers", type=int, default=0, help="layers per step (0 = the configuration's default)")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--pattern", choices=["fused", "reference"], default="fused",
                   help="launch sequence: the one lorax_amd.layers issues, or the reference caller's")
    p.add_argument("--no-plan", action="store_true", help="fused pattern without the host-built routing plan")
    p.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                   help="also run a plain device copy of MIB MiB (3 times) so that a counter run holds a kernel of "
                        "known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    p.add_argument("--two-launch", action="store_true",
                   help="fused pattern without the single-launch shrink+expand kernel for ranks 8 and 16")
    p.add_argument("--eager", action="store_true", help="launch every step eagerly instead of replaying a graph")
    p.add_argument("--no-tiles", action="store_true",
                   help="prefill launches search their row tiles on the device instead of taking the tables' plans")
    p.add_argument("--no-ceiling", action="store_true", help="skip the plain-torch copy / small-launch measurements")
    return p.parse_args()


DEFAULT_LAYERS = {"1": 32, "2": 32, "3": 8, "4": 2, "5": 1, "mid": 16, "5dec": 1, "2stk": 32}
# seconds of host time the CPU baseline of each configuration may take in the default run
CPU_BUDGET_S = {"1": 2.0, "2": 5.0, "3": 5.0, "4": 6.0, "5": 6.0, "mid": 2.0, "5dec": 4.0, "2stk": 2.0}
GATED = ("1", "2", "3", "4")  # configurations whose roofline fractions feed roofline_min


def build_workload(cfg: str, layers: int, device):
    from lorax_amd import synthetic

    L = layers or DEFAULT_LAYERS[cfg]
    if cfg == "mid":
        return synthetic.mid_prefill(device, num_layers=L, weights_on_device=True)
    if cfg == "5dec":
        return synthetic.config5_decode(device, num_layers=L, weights_on_device=True)
    if cfg == "2stk":
        # configuration 2 served from stacked weights ([num_adapters, r, h] tensors per layer and projection,
        # one entry number per token): the reference's path for preloaded adapters (utils/layers.py:79-105)
        w = synthetic.config2(device, num_layers=L, weights_on_device=True)
        w.name = "cfg2_bgmv_decode_qkvo_stacked_weights"
        w.stacked = True
        return w
    return synthetic.CONFIGS[int(cfg)](device, num_layers=L, weights_on_device=True)


class Plan:
    """Pre-built kernel arguments of one workload: per projection group the rank groups' tables plus the
    static v and y buffers, and closures that issue the launches of ONE layer in order.

    pattern "fused" is what lorax_amd.layers issues: in decode one batched shrink launch and one batched
    expand launch per projection group and rank; in prefill a shrink per projection group and rank (up to a
    summed rank of 128 per launch) and an expand per projection and rank.  The shrinks overwrite v, so there
    is no zero-fill in either.  pattern "reference" is the reference
    caller's sequence (utils/layers.py:114-164): zero-fill, shrink, expand for every projection and rank.
    """

    def __init__(self, w, pattern="fused", use_plan=True, fuse_small_ranks=True, use_tiles=True):
        import torch

        from lorax_amd import _native
        from lorax_amd.adapters import LORA

        self.w = w
        self.pattern = pattern
        self.use_plan = use_plan
        self.fuse_small_ranks = fuse_small_ranks
        self.use_tiles = use_tiles  # prefill launches take the tables' host-built row-tile plans
        self.batch = w.batch_data()
        self.calls = []  # (kind, fn(layer), algorithmic bytes, flops, gather bytes: weights once per routed row)
        T = w.num_tokens
        if getattr(w, "stacked", False):
            self._add_stacked(w)
            return
        for group in w.groups:
            x = w.inputs[group.name]
            y = torch.zeros((T, group.h_out), dtype=w.dtype, device=w.device)
            jobs = []  # (use_sgmv, r, rank_segments, offset, width)
            off = 0
            for name, size in zip(group.layer_names, group.sizes):
                data = self.batch.data.get(name, {}).get(LORA)
                if data is not None:
                    for r, rd in data.rank_data.items():
                        jobs.append((data.use_sgmv, r, rd, off, size))
                off += size
            decode = defaultdict(list)
            prefill = defaultdict(list)  # (rank, segment tables) -> [(rank_segments, offset, width)]
            for use_sgmv, r, rd, off, size in jobs:
                if use_sgmv:
                    from lorax_amd import sgmv

                    if (pattern == "fused" and rd.segments_key is not None
                            and sgmv.resident_shrink_applies(r, group.h_in, T)):
                        prefill[(r, rd.segments_key)].append((rd, off, size))
                    else:
                        self._add_sgmv(x, y, off, size, group.h_in, r, rd)
                elif pattern == "reference":
                    self._add_bgmv_reference(x, y, off, size, group.h_in, r, rd)
                else:
                    decode[r].append((rd, off, size))
            # as lorax_amd.layers: projections of one rank and the same segment tables shrink in one launch
            for (r, _), same in prefill.items():
                if fuse_small_ranks and _native.sgmv_lora_fits(r, group.h_in, T):
                    for i in range(0, len(same), _native.MAX_FUSED_BGMV_PROBLEMS):
                        self._add_sgmv_fused(x, y, group.h_in, r, same[i:i + _native.MAX_FUSED_BGMV_PROBLEMS])
                    continue
                step = max(1, min(_native.MAX_SGMV_SHRINK_PROBLEMS, 128 // r))
                self._add_sgmv_group(x, y, group.h_in, r, same, step)
            all_jobs = [(r, rd, off, size) for r, rank_jobs in decode.items() for rd, off, size in rank_jobs]
            all_fused = bool(all_jobs) and self.use_plan and self.fuse_small_ranks and all(
                _native.bgmv_lora_fits(r, group.h_in, size) for r, _, _, size in all_jobs)
            if all_fused:
                for r, rank_jobs in decode.items():
                    for i in range(0, len(rank_jobs), _native.MAX_FUSED_BGMV_PROBLEMS):
                        self._add_bgmv_fused(x, y, group.h_in, [(r,) + j for j in rank_jobs[i:i + 4]], True)
            else:
                step = _native.MAX_BGMV_PROBLEMS
                for i in range(0, len(all_jobs), step):
                    self._add_bgmv_fused(x, y, group.h_in, all_jobs[i:i + step], False)

    @staticmethod
    def _bgmv_counts(rd):
        routed = rd.indices >= 0
        rows = int(routed.sum().item())
        uniq = len(set(rd.lora_a_ptr[rd.indices[routed]].tolist()))
        return rows, uniq

    def _add_sgmv(self, x, y, off, size, h_in, r, rd):
        import torch

        from lorax_amd import sgmv

        e = 2
        v = torch.zeros((x.size(0), r), dtype=x.dtype, device=x.device)
        lens = (rd.segment_ends - rd.segment_starts).clamp(min=0)
        rows = int(lens.sum().item())
        uniq = len(set(rd.lora_a_t_ptr[lens > 0].tolist()))
        starts, ends, tmp_s, tmp_e = rd.segment_starts, rd.segment_ends, rd.tmp_shrink, rd.tmp_expand
        fused = self.pattern == "fused"
        resident_a = fused and sgmv.resident_shrink_applies(r, h_in)
        # the layers' pattern reads the resident stacks; the reference pattern its prefill layouts
        a_ptr = rd.lora_a_t_ptr if resident_a else rd.lora_a_ptr
        b_ptr = None if fused else rd.lora_b_ptr
        bt_ptr = rd.lora_b_t_ptr if fused else None
        a_is_rh = resident_a or not sgmv.use_cutlass_shrink(r)
        if a_is_rh:
            tmp_s = sgmv.get_shrink_scratch(x.device) if resident_a else sgmv.get_tmp_tensor(x.device)

        whole = rd.num_long_segments == starts.numel()  # the tables' row-tile plans cover the long segments
        shrink_tiles = rd.shrink_tiles if (fused and whole and self.use_tiles) else None
        expand_tiles = rd.expand_tiles if (fused and whole and self.use_tiles) else None

        def shrink(layer):
            if resident_a:  # overwrites the segments' rows of v: no zero-fill in this pattern
                sgmv._kernels.sgmv_shrink_multi([v], x, [a_ptr], starts, ends, tmp_s, layer, 1.0, False, shrink_tiles)
            elif a_is_rh:
                sgmv._kernels.sgmv_shrink(v, x, a_ptr, starts, ends, tmp_s, layer)
            else:
                sgmv._kernels.sgmv_cutlass(v, x, a_ptr, starts, ends, tmp_s, layer)

        def expand(layer):
            if bt_ptr is not None:
                sgmv.lora_b_sgmv_cutlass_slice(y, v, tmp_e, bt_ptr, starts, ends, layer, off, size, transposed=True,
                                               tiles=expand_tiles)
            else:
                sgmv.lora_b_sgmv_cutlass_slice(y, v, tmp_e, b_ptr, starts, ends, layer, off, size)

        if not resident_a:
            self.calls.append(("zero", lambda layer: v.zero_(), 0, 0, 0))
        self.calls.append(("sgmv_shrink", shrink, rows * h_in * e + uniq * r * h_in * e + rows * r * e,
                           2 * rows * r * h_in, rows * h_in * e + rows * r * h_in * e + rows * r * e))
        self.calls.append(("sgmv_expand", expand, rows * r * e + uniq * r * size * e + 2 * rows * size * e,
                           2 * rows * r * size, rows * r * e + rows * r * size * e + 2 * rows * size * e))

    def _add_sgmv_group(self, x, y, h_in, r, jobs, step):
        """Projections of one rank with the same segment tables, as lorax_amd.layers runs them: shrinks of `step`
        projections per launch (x counted once per launch; they overwrite v, no zero-fill), then one expand per
        projection from the resident B^T stacks.  Where the tables list many segments of a few rows last and carry
        a routing plan for them (decode tokens inside a prefill batch), the segment kernels take the long segments
        and ONE batched per-token shrink and ONE batched per-token expand take the rest, for all projections."""
        import torch

        from lorax_amd import _native, sgmv

        e = 2
        first = jobs[0][0]
        plans = [rd.short_plan for rd, _, _ in jobs]
        split = all(p is not None for p in plans)
        n_long = first.num_long_segments if split else first.segment_starts.numel()
        starts, ends = first.segment_starts[:n_long], first.segment_ends[:n_long]
        planned = self.use_tiles and n_long == first.num_long_segments
        shrink_tiles = first.shrink_tiles if planned else None
        expand_tiles = first.expand_tiles if planned else None
        lens = (ends - starts).clamp(min=0)
        rows = int(lens.sum().item())
        flat = torch.zeros((len(jobs), x.size(0), r), dtype=x.dtype, device=x.device)
        vs = list(flat.unbind(0))
        tmp_s = sgmv.get_shrink_scratch(x.device)
        for i in range(0, len(jobs), step):
            tables = [rd.lora_a_t_ptr[:n_long] for rd, _, _ in jobs[i:i + step]]
            shrink_bytes = shrink_gather = rows * h_in * e
            for table in tables:
                uniq = len(set(table[lens > 0].tolist()))
                shrink_bytes += uniq * r * h_in * e + rows * r * e
                shrink_gather += rows * r * h_in * e + rows * r * e

            def shrink(layer, out=vs[i:i + step], tables=tables):
                _native.sgmv_shrink_multi(out, x, tables, starts, ends, tmp_s, layer, 1.0, False, shrink_tiles)

            self.calls.append(("sgmv_shrink", shrink, shrink_bytes, 2 * rows * r * h_in * len(tables), shrink_gather))
        if split:
            # rows and distinct adapters of the plan: record = [count, 4 rows, A address, B address, 0]
            counts = [(int(p[:, 0].sum().item()), len(set(p[:, 5].tolist()))) for p in plans]
            n0 = counts[0][0]
            self.calls.append((
                "bgmv_shrink",
                lambda layer: _native.bgmv_multi([(v, x, None, None, 0, None) for v in vs], layer, 1.0, False, plans),
                n0 * h_in * e + sum(u * r * h_in * e + n * r * e for n, u in counts),
                sum(2 * n * r * h_in for n, _ in counts),
                n0 * h_in * e + sum(n * r * h_in * e + n * r * e for n, _ in counts)))
        for v, (rd, off, size) in zip(vs, jobs):
            b_table = rd.lora_b_t_ptr[:n_long]
            tmp_e = rd.tmp_expand[: sgmv.get_tmp_expand_size(n_long)]
            uniq = len(set(b_table[lens > 0].tolist()))

            def expand(layer, v=v, b_table=b_table, tmp_e=tmp_e, off=off, size=size):
                sgmv.lora_b_sgmv_cutlass_slice(y, v, tmp_e, b_table, starts, ends, layer, off, size, transposed=True,
                                               tiles=expand_tiles)

            self.calls.append(("sgmv_expand", expand, rows * r * e + uniq * r * size * e + 2 * rows * size * e,
                               2 * rows * r * size, rows * r * e + rows * r * size * e + 2 * rows * size * e))
        if split:
            problems = [(y, v, None, None, off, size) for v, (_, off, size) in zip(vs, jobs)]
            sizes = [size for _, _, size in jobs]
            self.calls.append((
                "bgmv_expand", lambda layer: _native.bgmv_multi(problems, layer, 1.0, True, plans),
                sum(n * r * e + u * r * size * e + 2 * n * size * e for (n, u), size in zip(counts, sizes)),
                sum(2 * n * r * size for (n, _), size in zip(counts, sizes)),
                sum(n * r * e + n * r * size * e + 2 * n * size * e for (n, _), size in zip(counts, sizes))))

    def _add_sgmv_fused(self, x, y, h_in, r, jobs):
        """Shrink and expand of up to four projections of a short prefill batch in one launch; v stays on chip."""
        from lorax_amd import _native

        e = 2
        first = jobs[0][0]
        starts, ends = first.segment_starts, first.segment_ends
        lens = (ends - starts).clamp(min=0)
        rows = int(lens.sum().item())
        problems = [(y, rd.lora_a_t_ptr, rd.lora_b_t_ptr, off, size) for rd, off, size in jobs]
        nbytes = gather = rows * h_in * e
        flops = 0
        for rd, _, size in jobs:
            uniq = len(set(rd.lora_a_t_ptr[lens > 0].tolist()))
            nbytes += uniq * r * (h_in + size) * e + 2 * rows * size * e
            gather += rows * r * (h_in + size) * e + 2 * rows * size * e
            flops += 2 * rows * r * (h_in + size)
        self.calls.append(("sgmv_lora", lambda layer: _native.sgmv_lora_multi(problems, x, starts, ends, r, layer),
                           nbytes, flops, gather))

    def _add_stacked(self, w):
        """The decode step over stacked weights: per projection group one PunicaWrapper.add_lora_slices call, which
        runs shrink and expand of the group's slices in one launch from the step's routing plan over stack entries.
        Same algorithmic bytes as the pointer-table launches of the same batch."""
        import torch

        from lorax_amd.adapters import LORA, stack_preloaded_adapters
        from lorax_amd.punica_wrapper import PunicaWrapper
        from lorax_amd.synthetic import make_meta

        e = 2
        adapters = sorted(w.rank_of_adapter)
        entry_of = {a: i for i, a in enumerate(adapters)}
        stacks = stack_preloaded_adapters(w.weights, adapters, w.device)
        wrapper = PunicaWrapper(max(w.num_tokens, 1), max(w.num_tokens, 1), str(w.device), enabled=True)
        # adapter 0 is the base model on this path: entry i belongs to adapter index i + 1
        wrapper.update_metadata(make_meta([entry_of[a] + 1 if a in entry_of else 0 for a in w.adapter_indices],
                                          w.device), prefill=False)
        self.keep = (stacks, wrapper)
        T = w.num_tokens
        for group in w.groups:
            x = w.inputs[group.name]
            y = torch.zeros((T, group.h_out), dtype=w.dtype, device=w.device)
            nbytes = gather = flops = 0
            x_counted = False
            off = 0
            spans = []
            for name, size in zip(group.layer_names, group.sizes):
                data = self.batch.data.get(name, {}).get(LORA)
                spans.append((name, off, size))
                off += size
                if data is None:
                    continue
                for r, rd in data.rank_data.items():
                    n, u = self._bgmv_counts(rd)
                    if not x_counted:
                        routed = int(sum(1 for a in w.adapter_indices if a in entry_of))
                        nbytes += routed * group.h_in * e
                        gather += routed * group.h_in * e
                        x_counted = True
                    nbytes += u * r * (group.h_in + size) * e + 2 * n * size * e
                    gather += n * r * (group.h_in + size) * e + 2 * n * size * e
                    flops += 2 * n * r * (group.h_in + size)

            def step(layer, x=x, y=y, spans=spans):
                wrapper.add_lora_slices(y, x, [stacks[(name, layer)] + (first, size) for name, first, size in spans], 1.0)

            self.calls.append(("bgmv_lora", step, nbytes, flops, gather))

    def _add_bgmv_reference(self, x, y, off, size, h_in, r, rd):
        import torch

        from lorax_amd import sgmv

        e = 2
        v = torch.zeros((x.size(0), r), dtype=x.dtype, device=x.device)
        rows, uniq = self._bgmv_counts(rd)
        idx, a_ptr, b_ptr = rd.indices, rd.lora_a_ptr, rd.lora_b_ptr
        self.calls.append(("zero", lambda layer: v.zero_(), 0, 0, 0))
        self.calls.append(("bgmv_shrink", lambda layer: sgmv.add_lora_a_bgmv(v, x, a_ptr, idx, layer),
                           rows * h_in * e + uniq * r * h_in * e + rows * r * e, 2 * rows * r * h_in,
                           rows * h_in * e + rows * r * h_in * e + rows * r * e))
        self.calls.append(("bgmv_expand",
                           lambda layer: sgmv.add_lora_b_bgmv_slice(y, v, b_ptr, idx, layer, off, size),
                           rows * r * e + uniq * r * size * e + 2 * rows * size * e, 2 * rows * r * size,
                           rows * r * e + rows * r * size * e + 2 * rows * size * e))

    def _add_bgmv_fused(self, x, y, h_in, jobs, single_launch):
        """jobs: (rank, rank_segments, column offset, width); one rank for the single launch, any mix otherwise."""
        import torch

        from lorax_amd import _native

        e = 2
        vs = [torch.zeros((x.size(0), r), dtype=x.dtype, device=x.device) for r, _, _, _ in jobs]
        shrink_problems = [(v, x, rd.lora_a_ptr, rd.indices, 0, None) for v, (_, rd, _, _) in zip(vs, jobs)]
        expand_problems = [(y, v, rd.lora_b_ptr, rd.indices, off, size) for v, (_, rd, off, size) in zip(vs, jobs)]
        counts = [self._bgmv_counts(rd) for _, rd, _, _ in jobs]
        any_routed = torch.stack([rd.indices >= 0 for _, rd, _, _ in jobs]).any(0)
        x_rows = int(any_routed.sum().item())  # the shared input is read once per launch
        shrink_bytes = x_rows * h_in * e + sum(u * r * h_in * e + n * r * e for (n, u), (r, _, _, _) in zip(counts, jobs))
        expand_bytes = sum(n * r * e + u * r * size * e + 2 * n * size * e
                           for (n, u), (r, _, _, size) in zip(counts, jobs))
        shrink_gather = x_rows * h_in * e + sum(n * r * h_in * e + n * r * e for (n, _), (r, _, _, _) in zip(counts, jobs))
        expand_gather = sum(n * r * e + n * r * size * e + 2 * n * size * e
                            for (n, _), (r, _, _, size) in zip(counts, jobs))
        plans = [rd.plan for _, rd, _, _ in jobs] if self.use_plan else None
        if single_launch:
            r = jobs[0][0]
            lora_problems = [(y, x, rd.plan, off, size) for _, rd, off, size in jobs]
            # v stays on chip: its write by the shrink and read by the expand are not memory traffic
            v_bytes = sum(2 * n * r * e for n, _ in counts)
            self.calls.append(("bgmv_lora", lambda layer: _native.bgmv_lora_multi(lora_problems, r, layer),
                               shrink_bytes + expand_bytes - v_bytes,
                               sum(2 * n * r * (h_in + size) for (n, _), (_, _, _, size) in zip(counts, jobs)),
                               shrink_gather + expand_gather - v_bytes))
            return
        self.calls.append(("bgmv_shrink", lambda layer: _native.bgmv_multi(shrink_problems, layer, 1.0, False, plans),
                           shrink_bytes, sum(2 * n * r * h_in for (n, _), (r, _, _, _) in zip(counts, jobs)),
                           shrink_gather))
        self.calls.append(("bgmv_expand", lambda layer: _native.bgmv_multi(expand_problems, layer, 1.0, True, plans),
                           expand_bytes,
                           sum(2 * n * r * size for (n, _), (r, _, _, size) in zip(counts, jobs)), expand_gather))

    def issue(self, layers, kinds=None):
        n = 0
        for layer in range(layers):
            for kind, fn, *_ in self.calls:
                if kinds is None or kind in kinds:
                    fn(layer)
                    n += 1
        return n

    def bytes_per_layer(self, kind=None):
        return sum(c[2] for c in self.calls if kind is None or c[0] == kind)

    def gather_bytes_per_layer(self, kind=None):
        return sum(c[4] for c in self.calls if kind is None or c[0] == kind)

    def launches_per_layer(self, kind=None):
        return sum(1 for c in self.calls if kind is None or c[0] == kind)


def capture(plan, layers, kinds=None):
    import torch

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        plan.issue(1, kinds)  # warm up lazily-initialised state outside the capture
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        n = plan.issue(layers, kinds)
    return graph, n


def time_graph(graph, reps, warmup=3, windows=5):
    """Duration of one replay in ms (median and best over `windows` windows of `reps` replays), from events
    recorded on the stream the replays run on."""
    import torch

    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(windows):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            graph.replay()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end) / reps)
    return statistics.median(times), min(times)


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(w, budget_s=5.0):
    """The reference's per-adapter masked matmul loop (oracle) on the host cores: one layer of the same
    batch, every projection; the adapter set is cut to a prefix if the full loop would blow the budget
    and the time is scaled linearly (the loop is linear in the number of adapters)."""
    import torch

    from oracle import lora_oracle as O

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    idx = torch.tensor(w.adapter_indices)
    active = sorted({a for a in w.adapter_indices if a in w.rank_of_adapter})
    xs = {g.name: w.inputs[g.name].cpu() for g in w.groups}

    def run(adapters, groups):
        compute = 0.0
        for g in groups:
            result = torch.zeros((w.num_tokens, g.h_out), dtype=w.dtype)
            off = 0
            for name, size in zip(g.layer_names, g.sizes):
                layer = w.weights[name].adapter_weights
                la = {a: layer[a].weights_a[:1].cpu() for a in adapters if a in layer}
                lb = {a: layer[a].weights_b[:1].cpu() for a in adapters if a in layer}
                t1 = time.perf_counter()
                O.fallback_layer_type(result, xs[g.name], idx, adapters, la, lb, 0, off, off + size)
                compute += time.perf_counter() - t1
                off += size
        return compute

    smallest = min(w.groups, key=lambda g: g.h_in * g.h_out)
    run(active[:1], [smallest])  # warm-up of the thread pool and the matmul kernels
    per_adapter = run(active[:1], w.groups)
    left = budget_s - per_adapter
    n = max(1, min(len(active), int(left / max(per_adapter, 1e-9))))
    times = [per_adapter] if n == 1 else []
    repeats = 3 if n == len(active) and 3 * n * per_adapter <= left else 1
    if n > 1:
        times = [run(active[:n], w.groups) for _ in range(repeats)]
    t_layer = statistics.median(times) * (len(active) / n)
    note = f"{n} of {len(active)} active adapters, 1 layer, all projections"
    if n < len(active):
        note += " (time extrapolated linearly in the adapter count)"
    return {
        "value": w.num_tokens / t_layer,
        "unit": "tokens/s per LoRA layer",
        "cores": torch.get_num_threads(),
        "os_cpu_count": os.cpu_count(),
        "cpu_model": cpu_model(),
        "kind": "port",
        "sample": note,
        "extrapolated": n < len(active),
        "seconds_per_layer": t_layer,
    }


def sig(x, digits=4):
    """x rounded to `digits` significant digits (keeps the JSON line short)."""
    if x is None or isinstance(x, (bool, int, str)):
        return x
    if x == 0 or x != x:
        return x
    from math import floor, log10

    return round(x, digits - 1 - int(floor(log10(abs(x)))))


def measure_ceiling(device, reps=10):
    """What plain torch operations reach on this GPU, as graph nodes timed like the kernels: a 1 GiB copy, a copy
    that moves 32 MiB, and a one-element kernel."""
    import torch

    def graph_of(fn, n):
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            fn(0)
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(n):
                fn(i)
        return g

    big = 1 << 30
    src = torch.ones(big, dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    g = graph_of(lambda i: dst.copy_(src), 4)
    ms, _ = time_graph(g, reps=reps, windows=3)
    copy_gbps = 2 * big * 4 / (ms * 1e-3) / 1e9
    del g, src, dst
    torch.cuda.empty_cache()
    small = 16 << 20
    pairs = 16  # 512 MiB of buffers: beyond the 256 MB memory-side cache
    bufs = torch.ones((2 * pairs, small), dtype=torch.uint8, device=device)
    g = graph_of(lambda i: bufs[2 * (i % pairs) + 1].copy_(bufs[2 * (i % pairs)]), 4 * pairs)
    ms, _ = time_graph(g, reps=reps, windows=3)
    copy32_us = ms * 1e3 / (4 * pairs)
    del g, bufs
    torch.cuda.empty_cache()
    one = torch.zeros(1, dtype=torch.float32, device=device)
    g = graph_of(lambda i: one.add_(1.0), 200)
    ms, _ = time_graph(g, reps=reps, windows=3)
    node_us = ms * 1e3 / 200
    del g
    return {
        "copy_1GiB_GBps": sig(copy_gbps), "copy_1GiB_frac_of_peak": sig(copy_gbps / HBM_PEAK_GBS),
        "copy_32MiB_moved_us": sig(copy32_us), "copy_32MiB_moved_GBps": sig(2 * small / (copy32_us * 1e-6) / 1e9),
        "small_launch_us": sig(node_us),
        "how": "torch copy_/add_ as HIP-graph nodes, events on the launch stream; GB/s = (read + written bytes) / time",
    }


def run_config(cfg: str, args, device):
    """Builds one configuration, times K steps (and further windows of K steps), times every kernel kind on its
    own and inside the step, and returns the configuration's record."""
    import torch

    w = build_workload(cfg, args.layers, device)
    L = w.num_layers
    plan = Plan(w, args.pattern, not args.no_plan, not args.two_launch, not args.no_tiles)
    torch.cuda.synchronize()

    if args.eager:
        run_step = lambda: plan.issue(L)  # noqa: E731
    else:
        graph, _ = capture(plan, L)
        run_step = graph.replay

    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    window_ms = []
    for _ in range(max(1, args.windows)):
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run_step()
        torch.cuda.synchronize()
        window_ms.append((time.perf_counter() - t0) * 1e3 / args.steps)
    first_ms = window_ms[0]  # exactly K steps after W warm-up steps: the figure of the top-level line
    median_ms = statistics.median(window_ms)

    # per-kernel timing over the same layer sweep: graphs that hold only one kind of launch ("us"), and the whole
    # step without that kind ("in_step_us" = what the kind adds to the step)
    kinds = sorted({c[0] for c in plan.calls if c[0] != "zero"})
    reps = max(5, min(50, args.steps))
    windows = max(1, args.windows)
    per_kind = {}
    step_event_ms = None
    if not args.eager:
        step_event_ms, _ = time_graph(graph, reps=reps, windows=windows)
    traffic_all = {}
    traffic_file = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(traffic_file):
        traffic_all = json.load(open(traffic_file)).get(f"cfg{cfg}", {})
    for kind in kinds:
        g, n = capture(plan, L, kinds={kind})
        ms, _ = time_graph(g, reps=reps, windows=windows)
        del g
        in_step_ms = ms
        others = {k for k in kinds if k != kind} | ({"zero"} if any(c[0] == "zero" for c in plan.calls) else set())
        if step_event_ms is not None:
            if others:
                g, _ = capture(plan, L, kinds=others)
                without_ms, _ = time_graph(g, reps=reps, windows=windows)
                del g
                in_step_ms = step_event_ms - without_ms
            else:
                in_step_ms = step_event_ms
        launches = plan.launches_per_layer(kind)
        bytes_per_launch = plan.bytes_per_layer(kind) / launches
        in_step_us = in_step_ms * 1e3 / n
        per_kind[kind] = {
            "n": launches,
            "MB": bytes_per_launch / 1e6,
            "us": ms * 1e3 / n,
            "in_step_us": in_step_us,
            "GBps": bytes_per_launch / (in_step_us * 1e-6) / 1e9,
            "frac": bytes_per_launch / (in_step_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "gather_GBps": plan.gather_bytes_per_layer(kind) / launches / (in_step_us * 1e-6) / 1e9,
            "traffic": traffic_all.get(kind),
            "share_ms": in_step_ms,
        }
    dominant = max(per_kind, key=lambda k: per_kind[k]["share_ms"])
    dk = per_kind[dominant]
    # A launch whose algorithmic bytes would take less than the ~2 us a graph node costs at the HBM peak is
    # bound by launch latency whatever the kernel does.
    launch_bound = dk["MB"] * 1e6 / (HBM_PEAK_GBS * 1e9) < 1e-6

    lens = ""
    if w.prefill:
        segs = sum(1 for i, a in enumerate(w.adapter_indices) if i == 0 or a != w.adapter_indices[i - 1])
        lens = f" runs={segs}"
    record = {
        "workload": f"{w.name} T={w.num_tokens}{lens} adapters={w.distinct_adapters()}/{len(w.rank_of_adapter)}",
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f16",
        "value": w.num_tokens * L / (median_ms * 1e-3),
        "unit": "tokens/s per LoRA layer",
        "ms_per_step": median_ms,
        "ms_per_step_first_window": first_ms,
        "tokens": w.num_tokens,
        "layers_per_step": L,
        "launch": "eager" if args.eager else "hip_graph",
        "pattern": args.pattern,
        "launches_per_layer": plan.launches_per_layer(),
        "MB_per_layer": plan.bytes_per_layer() / 1e6,
        "step_GBps": plan.bytes_per_layer() * L / (median_ms * 1e-3) / 1e9,
        "roofline": {
            "bound": "launch" if launch_bound else "hbm",
            "kernel": dominant,
            "achieved": dk["GBps"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dk["frac"],
            "traffic": dk["traffic"],
            "avg_launch_us": dk["in_step_us"],
            "bytes_per_launch": dk["MB"] * 1e6,
        },
        "kernels": per_kind,
    }
    if not args.no_cpu_baseline:
        record["cpu_baseline"] = cpu_baseline(w, args.cpu_budget or CPU_BUDGET_S[cfg])
    else:
        record["cpu_baseline"] = None
    del plan, w
    if not args.eager:
        del graph, run_step
    torch.cuda.empty_cache()
    return record


def compact(record):
    """One configuration's record as it goes into the JSON line: 4 significant digits, short keys."""
    out = {
        "workload": record["workload"],
        "dtype": record["dtype"],
        "value": sig(record["value"]),
        "ms_per_step": sig(record["ms_per_step"]),
        "layers": record["layers_per_step"],
        "launches_per_layer": record["launches_per_layer"],
        "kernels": {k: {f: sig(v[f]) for f in ("n", "MB", "us", "in_step_us", "frac", "traffic")}
                    for k, v in record["kernels"].items()},
        "roofline": {k: sig(v) for k, v in record["roofline"].items() if k not in ("avg_launch_us", "bytes_per_launch")},
    }
    cb = record["cpu_baseline"]
    out["cpu_baseline"] = None if cb is None else {
        "value": sig(cb["value"]), "cores": cb["cores"], "kind": cb["kind"], "sample": cb["sample"]}
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; --gpus above 1 is not supported by this build", file=sys.stderr)
        sys.exit(2)
    import torch

    from lorax_amd import _native

    if not _native.available():
        raise RuntimeError(f"liblorax_hip.so is missing: {_native.load_error()}")
    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs a GPU")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    _native.init(device)

    if args.calibrate_copy:
        src = torch.ones(args.calibrate_copy << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    todo = ["2", "1", "3", "4", "5", "mid", "5dec", "2stk"] if args.config == "all" else [args.config]
    records = {}
    for cfg in todo:
        print(f"bench: configuration {cfg}", file=sys.stderr, flush=True)
        records[cfg] = run_config(cfg, args, device)
    head = records[todo[0]]  # cfg2 in the default run
    ceiling = None
    if not args.eager and not args.no_ceiling:
        print("bench: ceiling", file=sys.stderr, flush=True)
        ceiling = measure_ceiling(device)

    cb = head["cpu_baseline"]
    out = {
        "metric": "LoRA-layer tokens/sec (BGMV decode / SGMV prefill), HBM roofline fraction in 'roofline'",
        "value": sig(head["tokens"] * head["layers_per_step"] / (head["ms_per_step_first_window"] * 1e-3), 6),
        "unit": "tokens/s per LoRA layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sig(head["ms_per_step_first_window"], 6),
        "ms_per_step_median": sig(head["ms_per_step"], 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": head["workload"], "layers_per_step": head["layers_per_step"], "launch": head["launch"],
                   "pattern": head["pattern"], "launches_per_layer": head["launches_per_layer"],
                   "MB_per_layer": sig(head["MB_per_layer"]), "step_GBps": sig(head["step_GBps"])},
        "roofline": {k: sig(v, 5) for k, v in head["roofline"].items()},
        "cpu_baseline": None if cb is None else {
            "value": sig(cb["value"]), "unit": cb["unit"], "cores": cb["cores"], "kind": cb["kind"],
            "sample": cb["sample"], "cpu_model": cb["cpu_model"], "os_cpu_count": cb["os_cpu_count"]},
        "ceiling": ceiling,
    }
    if args.config == "all":
        out["configs"] = {f"cfg{k}": compact(records[k]) for k in todo if k not in ("mid", "5dec", "2stk")}
        out["extra"] = {"mid_prefill_1k": compact(records["mid"]), "cfg5_decode_tokens_bgmv": compact(records["5dec"]),
                        "cfg2_stacked_weights": compact(records["2stk"])}
        fracs = [(f"cfg{k}", kind, rec["frac"], records[k]["roofline"]["bound"])
                 for k in GATED for kind, rec in records[k]["kernels"].items()]
        lowest = min(fracs, key=lambda t: t[2])
        out["roofline_min"] = {"config": lowest[0], "kernel": lowest[1], "frac": sig(lowest[2]), "bound": lowest[3]}
        hbm = [t for t in fracs if t[3] == "hbm"]
        if hbm:
            lowest = min(hbm, key=lambda t: t[2])
            out["roofline_min_hbm_bound"] = {"config": lowest[0], "kernel": lowest[1], "frac": sig(lowest[2])}
    else:
        out["kernels"] = compact(head)["kernels"]
    print(json.dumps(out, separators=(",", ":")))


if __name__ == "__main__":
    main()
