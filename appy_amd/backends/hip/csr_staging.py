"""How launches over the rows of a CSR matrix are staged: rows sorted by length, elements grouped by the
stripe they read, and kept orders of the elements (row plans) with the inspector that builds them.  A mix-in
of :class:`codegen.Launch`."""
from __future__ import annotations

import ctypes as C
import dataclasses

import numpy as np

from ...frontend import loop_ir
from . import runtime as rt
from .device import scratch_limit
from .kernelgen import Spec, Unsupported
from .row_plans import (PLAN_GROUPS, PLANS_PER_LOOP, RowPlan, _live_plans, _plans_lock, deal_runs, plan_kernel_spec,
                        plan_split)


class CsrStaging:
    def _stage_binned(self, vals, arrays, lo, hi, spec):
        """The launches of a loop whose rows are sorted by the trip count of their simd loop first:
        clear the counters, sort (`bins`), the rows of all classes (`mixed`), and for long rows that
        gather from a large operand: cut them at the stripes of that operand (`plan`), run the parts
        (phase 1), fold the partial results and run the rest of the body (phase 2)."""
        loop, a, env = self.loop, self.loop.analysis, self.env
        n = hi - lo
        V = spec.vec
        thresholds = [V, 8 * V, 32 * V]
        widthlog = [0, 2, 4, 6]
        trip, _uniform = loop._estimate_trip(env, arrays, n)
        base = sum(1 for t in thresholds if trip > t)
        # what the last launch of this loop found in its classes, if it was about the same arrays (a hint: their
        # contents may have changed).  The class with most rows is the one to take in natural order; without
        # long rows last time, this launch sets nothing up for parts (long rows, if there are some after
        # all, then run whole).  Neither changes the order in which the terms of a row are added.
        hint_addr, hint = loop.hint(self.device)
        seen = [int(hint[k]) for k in range(5)] if self.loop.options.get("hip_hints", True) else [0] * 5
        ident = self._hint_identity(arrays, lo, hi) if a.grouping is not None else (lo, hi)
        known = loop._hint_key.get(self.device) == ident and seen[0] == 1 and sum(seen[1:]) == n and min(seen[1:]) >= 0
        loop._hint_key[self.device] = ident
        parts, stripe, cap = 0, 0, 0
        gather = a.ragged[1]
        if gather is not None:
            x = arrays[gather[0]]
            x_bytes = int(x.shape[0]) * a.arrays[gather[0]].ty.size
            if self.hw.pinned_stripes and x_bytes > self.hw.stripe_min_bytes:
                parts = min(64, 8 * -(-x_bytes // (8 * self.hw.stripe_bytes)))
                stripe = -(-int(x.shape[0]) // parts)
                thresholds[2] = max(thresholds[2], 32 * parts)       # 32 elements per part at least
                # rows longer than the threshold: no more of them than the streamed arrays have room for
                bound = max([int(arrays[nm].shape[0]) for _code, streamed in loop._simd_loops for nm in streamed
                             if arrays[nm].ndim == 1] or [0])
                cap = min(n, bound // thresholds[2] + 1) if bound else n
        if known:
            # (the thresholds follow from element sizes and the size of the gathered operand, so the classes
            #  of the hint are the classes of this launch whenever the hint is about these arrays)
            base = max(range(4), key=lambda c: seen[c + 1])
            if seen[4] == 0:
                parts, stripe, cap = 0, 0, 0
        reds = max(1, len(loop_ir.reductions_of(a.team_split)))
        # one buffer: counters | row lists of the four classes | part boundaries | row starts | partial results
        # header: 8 counters, 64 part loads (8 bytes each), and a second such block that the binning kernel
        # clears instead when it is not run to clear the first
        off_rows = 2048
        off_bnd = off_rows + 4 * 4 * n
        off_start = (off_bnd + 4 * (parts + 1) * cap + 255) // 256 * 256        # where each listed row starts (8 bytes)
        off_part = (off_start + 8 * cap + 255) // 256 * 256
        total = off_part + 8 * reds * parts * cap
        buf = loop.scratch(self.device, self.stream, total)
        if buf is None:
            return False
        self.bin = {
            "counts": buf, "load": buf + 32, "zero": buf + 1024, "rows": buf + off_rows, "m": n, "base": base, "threshold": thresholds,
            "widthlog": widthlog, "skip": cap if parts else 0, "bnd": buf + off_bnd, "rowstart": buf + off_start, "cap": cap, "stripe": stripe,
            "nrows": buf + 4 * 3, "hint": hint_addr, "tlo": thresholds[base - 1] if base > 0 else -(1 << 62),
            "thi": thresholds[base] if base < 3 else (1 << 62),
        }
        self.scratch_ptr = buf + off_part
        self.nsplit = parts
        common = dict(block=256, vec=V, restrict=spec.restrict, stream_loads=spec.stream_loads)
        bins = loop.kernel_for(Spec("team", block=1024, vec=1, width=1, restrict=spec.restrict, aux="bins"))
        seq = []
        # the counters are cleared by the binning kernel itself, run over an empty range
        self.bin["zero"] = buf
        seq.append((bins, self._argument_block(bins, vals, arrays, 0, 0), (1, 1, 1), (1024, 1, 1)))
        self.bin["zero"] = buf + 1024
        seq.append((bins, self._argument_block(bins, vals, arrays, lo, hi),
                    (max(1, min(512, -(-n // 4096))), 1, 1), (1024, 1, 1)))
        # a wavefront for every slot of the base class: the other classes follow in further passes of the grid
        # (uniform rows of 16: 0.927 ms, as without binning, against 0.936 ms with 16384 workgroups that loop)
        waves = -(-(n << widthlog[base]) // 64)
        seq.append((self.kernel, self._argument_block(self.kernel, vals, arrays, lo, hi),
                    (max(256, min(loop.options.get("hip_max_blocks") or (1 << 20), -(-waves // 4))), 1, 1), (256, 1, 1)))
        if parts:
            ts = 8
            while ts < parts:
                ts *= 2
            self.bin["rows"] = buf + off_rows + 4 * 3 * n         # the list of class 3
            plan = loop.kernel_for(Spec("team", width=ts, rows="list", parts=parts, aux="plan",
                                        **{**common, "vec": 1, "stream_loads": False}))
            first = loop.kernel_for(Spec("team", width=16, phase=1, rows="list", parts=parts, **common))
            last = loop.kernel_for(Spec("team", width=1, phase=2, rows="list", parts=parts, **common))
            seq.append((plan, self._argument_block(plan, vals, arrays, lo, hi),
                        (max(1, min(2048, -(-cap * ts // 256))), 1, 1), (256, 1, 1)))
            seq.append((first, self._argument_block(first, vals, arrays, lo, hi),
                        (max(8, min(2048, 8 * -(-cap * 16 // 256))), 1, 1), (256, 1, 1)))
            seq.append((last, self._argument_block(last, vals, arrays, lo, hi),
                        (max(1, min(1024, -(-cap // 256))), 1, 1), (256, 1, 1)))
        self.sequence = seq
        self.args, self.grid, self.block = seq[2][1], seq[2][2], seq[2][3]
        if known and not self.plan_pending and not loop._value_only and not self.small:
            self.seq_replay = ("hints", loop._scratch_gen, ident, tuple(seen))
        return True

    def _stage_grouped(self, vals, arrays, lo, hi, spec) -> bool:
        """The launches of a loop of short rows whose simd loop sums terms that gather from an operand
        larger than an L2: group the elements of every 256 rows by the stripe of the operand they read
        (`group`), run the groups, stripe s on XCD s mod 8, sums per row and stripe to the scratch buffer
        (`cells`), add the sums of a row and run the rest of the body (phase 2).  The grouping kernel
        checks that the rows' ranges follow one another (as those of a CSR matrix do); where they do
        not, it raises a flag, the kernels after it return at once, and the loop runs row by row.
        When the last launch has reported rows in the class of the longest, the same launch lists those
        rows (`bins`), leaves them out of the groups and runs them in parts cut at the stripes (`plan`,
        `parts`, `fold`).  False (nothing staged) when the launch does not qualify."""
        loop, a, env = self.loop, self.loop.analysis, self.env
        n = hi - lo
        g = a.grouping
        if g is None or self.capture is not None:
            # (a launch recorded into a graph keeps its rows sorted by length: this form clears its flag with a
            #  memory-set node, and those are kept out of graphs)
            return False
        V = spec.vec
        # The form of the launch follows from what the host knows of these arrays (their sizes).  What the last
        # launch of the loop reported about the lengths of the rows only prunes it: when that launch was about
        # these same arrays and found no row beyond the limit, the kernels for such rows - which would run
        # empty - are left out.  Both forms add the terms of a row in the same order.
        _addr, hint = loop.hint(self.device)
        seen = [int(hint[k]) for k in range(5)]
        ident = self._hint_identity(arrays, lo, hi)
        trusted = (loop.options.get("hip_hints", True) and loop._hint_key.get(self.device) == ident
                   and seen[0] == 1 and sum(seen[1:]) == n and min(seen[1:]) >= 0)
        long_rows = not trusted or seen[4] > 0
        shape = loop.grouped_shape(n, env, arrays, self.hw)
        if shape is None:
            return False
        parts, shift, entries = shape
        # rows per block (blocks of 512 rows where the kept rows hold 7 elements on average - the power-law matrix with
        # mean 16 - were measured slower: 0.780 ms against 0.745; there are half as many wavefronts to group them)
        R = int(loop.options.get("hip_group_rows") or 256)
        nblk = -(-n // R)
        common = dict(block=256, restrict=spec.restrict)
        # rows beyond this many elements are cut at the stripes of the gathered operand, the others have their elements
        # grouped (power-law matrix: 3.14 ms with 128, 3.05 with 256, 3.02 with 512, 3.09 with 1024)
        cut = max(32 * V, 64 * parts)
        try:
            group = loop.kernel_for(Spec("team", vec=1, width=64, parts=parts, aux="group", block_rows=R, skip_long=long_rows, **common))
            cells = loop.kernel_for(Spec("team", vec=1, width=64, parts=parts, aux="cells", block_rows=R, guard=1, **common))
            sums = loop.kernel_for(Spec("team", vec=V, width=1, phase=2, guard=1, skip_long=long_rows, **common))
            plain = loop._choose_spec(n, env, arrays, restrict=spec.restrict, listable=False, hw=self.hw)
            if plain.kind != "team" or plain.phase or plain.rows:
                raise Unsupported("no plain team kernel to fall back to")
            rest = loop.kernel_for(dataclasses.replace(plain, guard=2))
            if long_rows:
                ts = 8
                while ts < parts:
                    ts *= 2
                listed = dict(common, rows="list", parts=parts, guard=1)
                bins = loop.kernel_for(Spec("team", block=1024, vec=1, width=1, restrict=spec.restrict, aux="bins"))
                plan = loop.kernel_for(Spec("team", vec=1, width=ts, aux="plan", **listed))
                first = loop.kernel_for(Spec("team", vec=V, width=16, phase=1, stream_loads=spec.stream_loads, **listed))
                last = loop.kernel_for(Spec("team", vec=V, width=1, phase=2, stream_loads=spec.stream_loads, **listed))
        except Unsupported:
            loop._group_off = True
            return False
        reds = max(1, len(loop_ir.reductions_of(a.team_split)))
        cap = 0
        if long_rows:
            bound = max([int(arrays[nm].shape[0]) for _code, streamed in loop._simd_loops for nm in streamed
                         if arrays[nm].ndim == 1] or [0])
            cap = min(n, bound // cut + 1) if bound else n
        # one buffer: header (counters of the sorting kernel, the flag) | lists of rows by class | cuts of the long rows |
        # their starts | their partial results | where the cells start | the grouped elements | sums per row and stripe
        off_rows = 2048
        off_bnd = off_rows + (4 * 4 * n if long_rows else 0)
        off_start = (off_bnd + 4 * (parts + 1) * cap + 255) // 256 * 256
        off_long = (off_start + 8 * cap + 255) // 256 * 256
        off_desc = (off_long + 8 * reds * parts * cap + 255) // 256 * 256
        off_ent = (off_desc + 4 * (parts + 1) * nblk + 255) // 256 * 256
        off_part = (off_ent + 8 * entries + 255) // 256 * 256
        buf = loop.scratch(self.device, self.stream, off_part + 4 * parts * n)
        if buf is None:
            return False
        hint_addr, _ = loop.hint(self.device)
        if trusted:
            base = max(range(3), key=lambda c: seen[c + 1])
        else:
            trip, _uniform = loop._estimate_trip(env, arrays, n)
            base = sum(1 for t in (V, 8 * V) if trip > t)
        loop._hint_key[self.device] = ident
        self.bin = {"flag": buf + 1984, "desc": buf + off_desc, "ent": buf + off_ent, "shiftc": shift, "entries": entries,
                    # (one limit in every form: rows beyond it are cut at the stripes when the launch has kernels for
                    #  them, and reported by the grouping kernel when it has not)
                    "rowmax": cut, "hint": hint_addr,
                    "counts": buf, "load": buf + 32, "zero": buf + 1024, "rows": buf + off_rows, "m": n, "base": base,
                    "threshold": [V, 8 * V, cut], "bnd": buf + off_bnd, "rowstart": buf + off_start, "cap": cap,
                    "stripe": -(-int(arrays[g["x"]].shape[0]) // parts), "nrows": buf + 4 * 3}
        self.scratch_ptr = buf + off_part
        self.nsplit = parts
        # the flag starts at zero, and with it the counters of the sorting kernel
        seq = [(None, ((buf, 2048) if long_rows else (buf + 1984, 8)), None, None)]
        if long_rows:
            seq.append((bins, self._argument_block(bins, vals, arrays, lo, hi), (max(1, min(512, -(-n // 4096))), 1, 1), (1024, 1, 1)))
        seq.append((group, self._argument_block(group, vals, arrays, lo, hi), (max(1, min(1 << 20, -(-nblk // 4))), 1, 1), (256, 1, 1)))
        seq.append((cells, self._argument_block(cells, vals, arrays, lo, hi), (8 * max(1, min(8192, -(-nblk // 4))), 1, 1), (256, 1, 1)))
        args_of_cells = seq[-1]
        seq.append((sums, self._argument_block(sums, vals, arrays, lo, hi), (max(1, min(4096, -(-n // 256))), 1, 1), (256, 1, 1)))
        if long_rows:
            self.bin["rows"] = buf + off_rows + 4 * 3 * n         # the list of the longest class
            self.scratch_ptr = buf + off_long
            seq.append((plan, self._argument_block(plan, vals, arrays, lo, hi), (max(1, min(2048, -(-cap * ts // 256))), 1, 1), (256, 1, 1)))
            seq.append((first, self._argument_block(first, vals, arrays, lo, hi), (max(8, min(2048, 8 * -(-cap * 16 // 256))), 1, 1), (256, 1, 1)))
            seq.append((last, self._argument_block(last, vals, arrays, lo, hi), (max(1, min(1024, -(-cap // 256))), 1, 1), (256, 1, 1)))
        # (the kernel that runs the loop row by row when the input was refused: few workgroups that loop - it returns at
        #  once otherwise, and 65536 workgroups take 15 us to do that, 1024 take 3)
        seq.append((rest, self._argument_block(rest, vals, arrays, lo, hi),
                    (min(1024, loop.grid_for(plain, n, cus=self.hw.cus, kernel=rest, row_hint=loop.row_hint(n, env, arrays))), 1, 1), (plain.block, 1, 1)))
        self.sequence = seq
        self.kernel, self.spec = cells, cells.src.spec
        self.args, self.grid, self.block = args_of_cells[1], args_of_cells[2], args_of_cells[3]
        if trusted and not self.plan_pending and not loop._value_only and not self.small:
            # (these kernels read the arrays themselves at every launch: a call with the same tensors may repeat them as they
            #  are while the last launch reports the classes of rows that this form was chosen for)
            self.seq_replay = ("hints", loop._scratch_gen, ident, tuple(seen))
        return True

    def _hint_identity(self, arrays, lo, hi):
        """Names the arrays the lengths of the rows come from (address and shape, not contents): what a launch
        reports about the rows is only believed by a launch over the same arrays."""
        out = [lo, hi]
        for nm in self.loop.plan_arrays():
            v = arrays[nm]
            out.append((nm, v.ctypes.data if isinstance(v, np.ndarray) else v.data_ptr(), tuple(v.shape)))
        return tuple(out)

    def _plan_identity(self, arrays, lo, hi, vals):
        """``(key, tensors)`` naming the contents a row plan of this launch would describe, or None when
        they cannot be named: every array the plan reads must be a tensor on the GPU (its version counter
        tells of in-place changes)."""
        loop = self.loop
        names = loop.plan_arrays()
        tensors, key = [], [self.device, lo, hi, int(arrays[loop.analysis.grouping["x"]].shape[0])]
        for nm in names:
            t = arrays[nm]
            if isinstance(t, np.ndarray) or not getattr(t, "is_cuda", False) or not hasattr(t, "_version"):
                return None
            tensors.append(t)
            key.append((nm, t.data_ptr(), tuple(t.shape), tuple(t.stride()), t._version))
        for nm in loop.arg_names:
            if nm in loop.analysis.scalars:
                v = vals[nm]
                key.append((nm, v.item() if isinstance(v, np.generic) else v))
        return tuple(key), tensors

    def _stage_planned(self, vals, arrays, lo, hi, spec) -> bool:
        """The launches of a loop whose elements have been ordered by an earlier launch with the same arrays
        (a row plan): the kernel that runs the plan, then the kernel that adds the sums of a row's eight
        column ranges and runs the rest of the body.  A plan is built the second time a set of arrays is
        seen unchanged (`hip_reuse="now"`: the first time, `hip_reuse=k`: the k-th); before that the launch takes the forms that
        keep nothing.  False (nothing staged) when the launch does not qualify or has no plan yet."""
        loop, a, env = self.loop, self.loop.analysis, self.env
        reuse = loop.options.get("hip_reuse", True)
        if a.grouping is None or not reuse or loop._plan_off or self.capture is not None:
            # (a launch recorded into a graph is replayed without being staged again: it must read the arrays
            #  themselves every time, not an order worked out from what they held when it was recorded)
            return False
        n = hi - lo
        ident = self._plan_identity(arrays, lo, hi, vals)
        if ident is None:
            return False
        key, tensors = ident
        plan = None
        if any(not pl.valid for pl in loop._plans):
            # plans that a store into their arrays has made untrue: their memory goes back once the launches
            # that were queued with them have finished
            with loop._lock:
                dead = [pl for pl in loop._plans if not pl.valid]
                loop._plans = [pl for pl in loop._plans if pl.valid]
            rt.device_sync()
            for pl in dead:
                pl.release()
        with loop._lock:
            for cand in loop._plans:
                if cand.key == key and cand.alive(tensors):
                    plan = cand
                    loop._plans.remove(cand)
                    loop._plans.append(cand)
                    break
        if plan is None:
            if key in loop._plan_refused:
                return False
            shape = loop.plan_shape(n, env, arrays, self.hw)
            if shape is None:
                return False
            import weakref

            with loop._lock:
                # sightings of these very tensor objects (an address is handed out again once a tensor is freed)
                count, refs = loop._plan_seen.get(key, (0, ()))
                if not (len(refs) == len(tensors) and all(r() is t for r, t in zip(refs, tensors))):
                    count, refs = 0, tuple(weakref.ref(t) for t in tensors)
                seen = count + 1
                if len(loop._plan_seen) > 64:
                    loop._plan_seen.clear()
                loop._plan_seen[key] = (seen, refs)
            # the sighting at which the order is worked out: the second by default, the first with "now", the k-th with
            # an integer k (working it out costs some eight launches over the raw arrays: a program that knows it will
            # launch a few times only may ask for a later sighting, or switch the reuse off)
            wanted = 1 if reuse == "now" else (max(1, reuse) if isinstance(reuse, int) and not isinstance(reuse, bool) else 2)
            if seen < wanted:
                # (the next launch over these tensors may build a plan: this one must not be repeated in its place)
                self.plan_pending = True
                return False
            plan = self._build_plan(key, tensors, shape, vals, arrays, lo, hi, spec)
            if plan is None:
                return False
        V = spec.vec
        try:
            cells = loop.kernel_for(plan_kernel_spec(plan.tile, plan.entries, n, spec.restrict))
            sums = loop.kernel_for(Spec("team", block=256, vec=V, width=1, phase=2, guard=1, restrict=spec.restrict))
        except Unsupported:
            loop._plan_off = True
            return False
        self.bin = dict(plan.bin)
        split = plan.split
        self.bin["split"] = split
        self.scratch_ptr = loop.scratch(self.device, self.stream, 4 * PLAN_GROUPS * split * n)
        if self.scratch_ptr is None:
            return False
        self.nsplit = PLAN_GROUPS * split
        self.plan = plan
        seq = [(cells, self._argument_block(cells, vals, arrays, lo, hi), (plan.grid, 1, 1), (1024, 1, 1)),
               (sums, self._argument_block(sums, vals, arrays, lo, hi), (max(1, min(4096, -(-n // 256))), 1, 1), (256, 1, 1))]
        self.sequence = seq
        self.kernel, self.spec = cells, cells.src.spec
        self.args, self.grid, self.block = seq[0][1], seq[0][2], seq[0][3]
        if not loop._value_only and not self.small:
            # a call with these same tensors may repeat the two launches without staging them again, as long as the plan
            # stands (`CompiledLoop._sequence_still_right`)
            import weakref

            self.seq_replay = ("plan", loop._scratch_gen, plan,
                               [(loop.arg_names.index(nm), weakref.ref(t), t._version) for nm, t in zip(loop.plan_arrays(), tensors)])
        return True

    def _build_plan(self, key, tensors, shape, vals, arrays, lo, hi, spec):
        """Runs the inspector for these arrays: the generated kernel writes one (key, value) pair per element, the
        library sorts the pairs and lays out cells, tiles and slots.  Waits for the device after that kernel, to learn
        whether the arrays were accepted (row ranges that follow one another, indices inside the operand) and whether
        every position holds an element, and once more at the end."""
        loop = self.loop
        n = hi - lo
        try:
            rkeys = loop.kernel_for(Spec("team", block=256, vec=1, width=64, aux="rkeys", block_rows=256, restrict=spec.restrict))
        except Unsupported:
            loop._plan_off = True
            return None
        lib = rt.lib()
        temp_bytes, max_tiles, words = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
        rt.check(lib.appy_hip_rowplan_sizes(C.byref(shape), C.byref(temp_bytes), C.byref(max_tiles), C.byref(words)))
        entries = int(shape.entries)
        ncell = int(shape.row_blocks) * int(shape.groups)
        limit = scratch_limit(self.device)
        slack = 4 * int(shape.tile)      # the kernel that runs the plan reads whole tiles, a few beyond the end of a cell
        kept = 8 * (entries + slack) + 4 * (words.value + slack) + 8 * (ncell + 1) + 256
        if kept + 16 * entries + temp_bytes.value > limit:
            return None
        # older plans of this loop make room first (their launches have been queued before this one on their streams)
        with loop._lock:
            old = [pl for pl in loop._plans if not pl.valid] + [pl for pl in loop._plans if pl.valid][:-(PLANS_PER_LOOP - 1) or None]
            loop._plans = [pl for pl in loop._plans if pl not in old]
        if old:
            rt.device_sync()
            for pl in old:
                pl.release()
        import weakref

        plan = RowPlan(self.device, key, [weakref.ref(t) for t in tensors],
                       [(t.data_ptr(), t.numel() * t.element_size()) for t in tensors])
        temps = []
        t0 = t1 = None
        try:
            elements = plan.alloc(8 * (entries + slack))
            cstart = plan.alloc(4 * (ncell + 1))
            tbase = plan.alloc(4 * (ncell + 1))
            rstream = plan.alloc(4 * (words.value + slack))
            flag = plan.alloc(256)
            for nb in (4 * entries, 8 * entries, 4 * entries, temp_bytes.value):
                temps.append(rt.malloc(max(256, nb)))
            keys, pairs, keys_sorted, temp = temps
            rkeys_fn = rkeys.function(self.device)      # (loads the code object: not part of the inspector's time)
            t0, t1 = rt.Event(), rt.Event()
            t0.record(self.stream)
            rt.memset_async(keys, 0xFF, 4 * entries, self.stream)
            rt.memset_async(flag, 0, 256, self.stream)
            self.bin = {"keys": keys, "vals": pairs, "entries": entries, "nx": int(arrays[loop.analysis.grouping["x"]].shape[0]),
                        "lbits": int(shape.line_bits), "flag": flag}
            args = self._argument_block(rkeys, vals, arrays, lo, hi)
            nblk = -(-n // 256)
            rt.launch(rkeys_fn, (max(1, min(1 << 20, -(-nblk // 4))), 1, 1), (256, 1, 1), args, self.stream)
            # what the kernel found: whether the arrays are accepted, and how many positions the rows cover - all of them
            # (the usual case: a loop over all rows of a CSR matrix) means that the sort needs one pass less
            words = (C.c_int64 * 2)(0, 0)
            rt.memcpy_d2h(C.addressof(words), flag, 16, self.stream)      # waits for the stream
            word = C.c_int64(words[0])
            if not word.value:
                shape.full = 1 if words[1] == entries else 0
                rt.check(lib.appy_hip_rowplan_build(C.byref(shape), keys, pairs, keys_sorted, elements, temp, temp_bytes.value,
                                                    cstart, tbase, rstream, self.stream))
            t1.record(self.stream)
            rt.sync(self.stream)          # (the temporary arrays go back below)
            plan.inspector_ms = t0.elapsed_ms(t1)
        except BaseException:
            plan.release()
            raise
        finally:
            for ptr in temps:
                rt.free(ptr)
        if word.value:
            plan.release()
            loop._plan_refused.add(key)
            return None
        plan.bin = {"ent": elements, "cstart": cstart, "tbase": tbase, "rstream": rstream, "ncell": ncell,
                    "gwidth": int(shape.group_width), "colbits": int(shape.col_bits), "flag": flag,
                    "nx": int(arrays[loop.analysis.grouping["x"]].shape[0])}
        plan.ncell = ncell
        plan.tile = int(shape.tile)
        # few cells (a matrix of few blocks of rows): several workgroups share a cell, each with a run of its tiles,
        # until there are some four workgroups per compute unit or a workgroup is down to two tiles
        # how the tiles lie over the cells decides how many workgroups share a cell and which runs a workgroup gets
        tb = np.empty(ncell + 1, dtype=np.uint32)
        rt.memcpy_d2h(tb.ctypes.data, tbase, 4 * (ncell + 1), self.stream)
        tiles = np.diff(tb.astype(np.int64))
        plan.split = plan_split(tiles, self.hw.cus, plan.tile, entries, loop.options.get("hip_plan_split"))
        # one workgroup per CU (their LDS allows no more), a multiple of eight so that a workgroup stays with one column
        # range; each walks the tiles of its runs as one sequence
        grid = min(ncell * plan.split, int(loop.options.get("hip_plan_grid") or max(8, self.hw.cus // 8 * 8)))
        plan.grid = max(8, grid // 8 * 8)
        order = deal_runs(tiles, plan.split, plan.grid)
        try:
            dealt = plan.alloc(4 * len(order))
            rt.memcpy_h2d(dealt, order.ctypes.data, 4 * len(order), self.stream)
        except BaseException:
            plan.release()
            raise
        plan.bin["order"], plan.bin["norder"] = dealt, len(order)
        plan.entries = entries
        plan.valid = True
        plan.owner = loop
        with loop._lock:
            loop._plans.append(plan)
            # what the launches before this one needed on this stream (8 bytes per element for the grouped form) is
            # not needed by the launches that run the plan; the stream has just been waited for
            stale = loop._scratch.pop((self.device, self.stream), None)
            loop._scratch_gen += 1
        if stale is not None:
            rt.free(stale[0])
        with _plans_lock:
            _live_plans.append(plan)
        loop.last_plan = plan
        return plan
