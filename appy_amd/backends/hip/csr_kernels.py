"""Kernel bodies for loops over the rows of a CSR matrix that read the raw arrays at every launch:
rows binned by length (``bins``, ``mixed``, ``listed``) and elements grouped by the stripe of the
gathered operand they read (``group``, ``cells``).  A mix-in of :class:`kernelgen.KernelBuilder`,
whose statement lowering (``self.w``, ``self.block``, ``self._iteration`` ...) it uses."""
from __future__ import annotations

from ...frontend import loop_ir
from . import dtypes as T
from .exprs import cast, cname
from .loop_analysis import Unsupported


class CsrKernels:
    # ---- rows binned by the trip count of their simd loop ----------------------------------------
    # Classes: 0..3 by rising trip count (thresholds are kernel arguments).  The rows of one class,
    # the base class, are taken in their natural order; the rows of the others are listed by the
    # binning kernel: `__rows[c * __m + k]`, `__counts[c]` of them.
    def _split_iteration(self, idx_code: str, guard=None, upto=None):
        """One iteration, the scalar set-up first; ``guard`` (a C condition that may use
        ``__trip``, the trip count of the simd loop) decides whether the rest runs."""
        a = self.a
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        self.w("{")
        self.ind += 1
        self.w(f"const appy::i64 {cname(a.var)} = {idx_code};")
        self._declare_locals()
        self.block(body[:at])
        if guard is not None:
            lo, hi = self._range_args(a.team_split)
            self.w(f"const appy::i64 __trip = ({hi}) - ({lo});")
            self.w(f"if ({guard}) {{")
            self.ind += 1
        self.block(body[at:upto])
        if guard is not None:
            self.ind -= 1
            self.w("}")
        self.ind -= 1
        self.w("}")

    def _body_bins(self):
        """The kernel that sorts rows into classes: one lane per row runs the set-up, the rows of
        every class but the base class are appended to the list of their class (one reservation
        per workgroup, chunk and class).  It also clears the counters of the next launch."""
        RPT = 4
        B = self.spec.block
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.mode = "lane"
        self.w("__shared__ int __cnt[4];")
        self.w("__shared__ int __first[4];")
        self.w("if (blockIdx.x == 0 && threadIdx.x < 136) __zero[threadIdx.x] = 0;     // 8 counters, 64 part loads of 8 bytes")
        self.w(f"for (appy::i64 __c0 = __lo + (appy::i64)blockIdx.x * {B * RPT}; __c0 < __hi; __c0 += (appy::i64)gridDim.x * {B * RPT}) {{")
        self.ind += 1
        self.w("if (threadIdx.x < 4) __cnt[threadIdx.x] = 0;")
        self.w("__syncthreads();")
        self.w(f"int __cl[{RPT}], __pos[{RPT}];")
        self.w("#pragma unroll")
        self.w(f"for (int __r = 0; __r < {RPT}; ++__r) {{")
        self.ind += 1
        self.w(f"const appy::i64 __i = __c0 + (appy::i64)__r * {B} + threadIdx.x;")
        self.w("__cl[__r] = -1;")
        self.w("__pos[__r] = 0;")
        self.w("if (__i < __hi) {")
        self.ind += 1
        body = self.a.outer.body
        at = next(k for k, st in enumerate(body) if st is self.a.team_split)
        self.w(f"const appy::i64 {cname(var)} = __i;")
        self._declare_locals()
        self.block(body[:at])
        lo, hi = self._range_args(self.a.team_split)
        self.w(f"const appy::i64 __trip = ({hi}) - ({lo});")
        self.w("const int __c = __trip <= __t0 ? 0 : __trip <= __t1 ? 1 : __trip <= __t2 ? 2 : 3;")
        self.w("if (__c != __base) { __cl[__r] = __c; __pos[__r] = atomicAdd(&__cnt[__c], 1); }")
        self.ind -= 1
        self.w("}")
        self.ind -= 1
        self.w("}")
        self.w("__syncthreads();")
        self.w("if (threadIdx.x < 4) __first[threadIdx.x] = __cnt[threadIdx.x] ? atomicAdd(&__counts[threadIdx.x], __cnt[threadIdx.x]) : 0;")
        self.w("__syncthreads();")
        self.w("#pragma unroll")
        self.w(f"for (int __r = 0; __r < {RPT}; ++__r) {{")
        self.w(f"    if (__cl[__r] >= 0) __rows[(appy::i64)__cl[__r] * __m + __first[__cl[__r]] + __pos[__r]] = "
               f"(int)(__c0 + (appy::i64)__r * {B} + threadIdx.x);")
        self.w("}")
        self.w("__syncthreads();")
        self.ind -= 1
        self.w("}")

    def _body_mixed(self):
        """Rows of all classes in one kernel: the wavefronts walk a row of slots, first the rows of
        the base class in their natural order (rows of other classes are passed over), then the
        listed rows class by class; the team width of a wavefront follows the class of its slot."""
        NWB = self.spec.block // 64
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.w("const int __lid = threadIdx.x & 63;")
        self.w(f"const appy::i64 __wv = (appy::i64)blockIdx.x * {NWB} + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);")
        self.w(f"const appy::i64 __nwv = (appy::i64)gridDim.x * {NWB};")
        prev = "0"
        for c in range(4):
            skip = "__skip3" if c == 3 else "0"
            self.w(f"const appy::i64 __l{c} = (appy::i64)__counts[{c}] - {skip};")
            self.w(f"const appy::i64 __n{c} = (__base == {c}) ? (__hi - __lo) : (__l{c} > 0 ? __l{c} : 0);")
            self.w(f"const appy::i64 __e{c} = {prev} + (((__n{c} << __wl{c}) + 63) >> 6);")
            prev = f"__e{c}"
        # what the classes held this time, left where the host can see it when it stages the next launch
        # (a hint for shaping that launch: which class to take in natural order, whether long rows exist)
        self.w("if (blockIdx.x == 0 && threadIdx.x == 0) {")
        self.w("    const appy::i64 __others = (__base == 0 ? 0 : (appy::i64)__counts[0]) + (__base == 1 ? 0 : (appy::i64)__counts[1]) "
               "+ (__base == 2 ? 0 : (appy::i64)__counts[2]) + (__base == 3 ? 0 : (appy::i64)__counts[3]);")
        for c in range(4):
            self.w(f"    __hint[{c + 1}] = (__base == {c}) ? (__hi - __lo) - __others : (appy::i64)__counts[{c}];")
        self.w("    __hint[0] = 1;")
        self.w("}")
        self.w("for (appy::i64 __v = __wv; __v < __e3; __v += __nwv) {")
        self.ind += 1
        self.w("const int __c = (int)(__v >= __e0) + (int)(__v >= __e1) + (int)(__v >= __e2);")
        self.w("const int __wl = __c == 0 ? __wl0 : __c == 1 ? __wl1 : __c == 2 ? __wl2 : __wl3;")
        self.w("const int __W = 1 << __wl;")
        self.w("const int __lane = __lid & (__W - 1);")
        self.w("const appy::i64 __vb = __c == 0 ? 0 : __c == 1 ? __e0 : __c == 2 ? __e1 : __e2;")
        self.w("const appy::i64 __nc = __c == 0 ? __n0 : __c == 1 ? __n1 : __c == 2 ? __n2 : __n3;")
        self.w("const appy::i64 __t = ((__v - __vb) << (6 - __wl)) + (__lid >> __wl);")
        self.w("if (__t < __nc) {")
        self.ind += 1
        self.w("const appy::i64 __i = (__c == __base) ? (__lo + __t) : "
               "(appy::i64)__rows[(appy::i64)__c * __m + (__c == 3 ? __skip3 : 0) + __t];")
        self.mode = "team"
        self._split_iteration("__i", guard="__c != __base || (__trip > __tlo && __trip <= __thi)")
        self.mode = "lane"
        self.ind -= 1
        self.w("}")
        self.ind -= 1
        self.w("}")

    def _body_listed(self):
        """Kernels over the rows of one list whose simd loop runs in planned parts: the planning
        kernel, the kernel that runs the parts (part p on the workgroups whose number is p modulo 8:
        workgroups go to the eight XCDs in turn, so every L2 sees one stripe of the gathered
        operand), and the finishing kernel."""
        s = self.spec
        W, B, S = s.width, s.block, s.parts
        tpb = B // W
        var = self.a.var
        self.ex.locals[var] = T.WEAK_INT
        self.w(f"const int __lane = threadIdx.x & {W - 1};")
        self.w(f"const appy::i64 __team = threadIdx.x / {W};")
        self.w("const appy::i64 __listed = (appy::i64)__nrows[0];")
        self.w("const appy::i64 __n = __listed < __cap ? __listed : __cap;")
        if s.aux == "plan":
            x_name, idx_name = self.a.ragged[1]
            idx = self.a.arrays[idx_name]
            idx.loaded = True
            # elements per part over all rows: the kernel that runs the parts looks at these before it
            # ties parts to XCDs (columns that crowd into few stripes would leave most XCDs idle)
            self.w(f"__shared__ unsigned long long __work[{S}];")
            self.w(f"if (threadIdx.x < {S}) __work[threadIdx.x] = 0;")
            self.w("__syncthreads();")
            self.w("unsigned long long __mine = 0;      // elements in the part of this lane, over the rows of its team")
            self.w(f"for (appy::i64 __t = (appy::i64)blockIdx.x * {tpb} + __team; __t < __n; __t += (appy::i64)gridDim.x * {tpb}) {{")
            self.ind += 1
            self.mode = "team"
            self.w("{")
            self.ind += 1
            self.w(f"const appy::i64 {cname(var)} = (appy::i64)__rows[__t];")
            self._declare_locals()
            body = self.a.outer.body
            at = next(k for k, st in enumerate(body) if st is self.a.team_split)
            self.block(body[:at])
            lo, hi = self._range_args(self.a.team_split)
            self.w(f"const appy::i64 __rlo = {lo};")
            self.w(f"const appy::i64 __rhi = ({hi}) > __rlo ? ({hi}) : __rlo;")
            # lane p < S - 1 looks for the first position whose index reaches stripe p + 1; a running
            # maximum over the lanes keeps the cuts in order, so that every position lies in exactly
            # one part whatever the order of the indices (sorted rows are cut at the stripes)
            # (the search starts where the cut would lie if the indices were spread evenly and widens its steps from
            #  there - two or three cache lines of indices per cut instead of one per level of a bisection of the whole
            #  row; 0.14 ms of a 3 ms launch were these lines)
            self.w("appy::i64 __b = __rhi;")
            self.w(f"if (__lane < {S - 1} && __rhi > __rlo) {{")
            self.w("    const appy::i64 __target = (appy::i64)(__lane + 1) * __stripe;")
            self.w("    appy::i64 __a = __rlo, __z = __rhi;       // the cut lies in [__a, __z]: indices before __a are below the target")
            self.w(f"    const appy::i64 __guess = __rlo + ((__rhi - __rlo) * (__lane + 1)) / {S};")
            self.w("    appy::i64 __step = 16;")
            self.w(f"    if ((appy::i64){cname(idx_name)}[__guess] < __target) {{")
            self.w("        __a = __guess + 1;")
            self.w("        while (__a < __z) {")
            self.w("            const appy::i64 __p = (__a + __step - 1) < (__z - 1) ? (__a + __step - 1) : (__z - 1);")
            self.w(f"            if ((appy::i64){cname(idx_name)}[__p] < __target) {{ __a = __p + 1; __step *= 4; }} else {{ __z = __p; break; }}")
            self.w("        }")
            self.w("    } else {")
            self.w("        __z = __guess;")
            self.w("        while (__a < __z) {")
            self.w("            const appy::i64 __p = (__z - __step) > __a ? (__z - __step) : __a;")
            self.w(f"            if ((appy::i64){cname(idx_name)}[__p] < __target) {{ __a = __p + 1; break; }} else {{ __z = __p; __step *= 4; }}")
            self.w("        }")
            self.w("    }")
            self.w("    while (__a < __z) {")
            self.w("        const appy::i64 __mid = __a + ((__z - __a) >> 1);")
            self.w(f"        if ((appy::i64){cname(idx_name)}[__mid] < __target) __a = __mid + 1; else __z = __mid;")
            self.w("    }")
            self.w("    __b = __a;")
            self.w("}")
            self.w(f"__b = appy::team_running_max<{W}>(__b, __lane);")
            # (cuts are kept relative to the start of the row: 32 bits are enough whatever the array size)
            self.w("if (__lane == 0) { __bnd[__t] = 0; __start[__t] = __rlo; }")
            self.w(f"const appy::i64 __cut = (__lane < {S - 1} ? __b : __rhi) - __rlo;      // where part __lane ends")
            self.w(f"if (__lane < {S}) __bnd[(appy::i64)(__lane + 1) * __cap + __t] = (int)__cut;")
            self.w(f"const appy::i64 __before = appy::team_lane_below<{W}>(__cut, __lane);")
            self.w(f"if (__lane < {S} && __cut > (__lane ? __before : 0)) __mine += (unsigned long long)(__cut - (__lane ? __before : 0));")
            self.ind -= 1
            self.w("}")
            self.mode = "lane"
            self.ind -= 1
            self.w("}")
            self.w(f"if (__lane < {S} && __mine) atomicAdd(&__work[__lane], __mine);")
            self.w("__syncthreads();")
            self.w(f"if (threadIdx.x < {S} && __work[threadIdx.x]) atomicAdd(&__load[threadIdx.x], __work[threadIdx.x]);")
            return
        self.mode = "team"
        if s.phase == 1:
            # Part p of every row runs on the workgroups whose number is p modulo 8, i.e. on one XCD, whose L2
            # then holds stripe p of the gathered operand and nothing else of it.  That ties the work of an XCD
            # to the elements that fall into its stripes: when one XCD would get more than 1.5 times its share
            # (columns crowded into few stripes), the parts are dealt to all workgroups alike instead, stripe
            # after stripe.
            self.w("unsigned long long __tot = 0, __most = 0;")
            self.w("for (int __x = 0; __x < 8; ++__x) {")
            self.w("    unsigned long long __sum = 0;")
            self.w(f"    for (int __p = __x; __p < {S}; __p += 8) __sum += __load[__p];")
            self.w("    __tot += __sum;")
            self.w("    __most = __sum > __most ? __sum : __most;")
            self.w("}")
            self.w("const bool __even = __most * 16 <= __tot * 3;")
            self.w(f"const appy::i64 __t0 = (__even ? (appy::i64)(blockIdx.x >> 3) : (appy::i64)blockIdx.x) * {tpb} + __team;")
            self.w(f"const appy::i64 __dt = (__even ? (appy::i64)(gridDim.x >> 3) : (appy::i64)gridDim.x) * {tpb};")
            self.w(f"for (appy::i64 __pass = 0; __pass < (__even ? {S // 8} : {S}); ++__pass) {{")
            self.ind += 1
            self.w("const appy::i64 __chunk = __even ? (appy::i64)(blockIdx.x & 7) + 8 * __pass : __pass;")
            self.w("for (appy::i64 __t = __t0; __t < __n; __t += __dt) {")
            self.ind += 1
            body = self.a.outer.body
            at = next(k for k, st in enumerate(body) if st is self.a.team_split)
            self._split_iteration("(appy::i64)__rows[__t]", upto=at + 1)
            self.ind -= 1
            self.w("}")
            self.ind -= 1
            self.w("}")
        else:
            self.w(f"for (appy::i64 __t = (appy::i64)blockIdx.x * {tpb} + __team; __t < __n; __t += (appy::i64)gridDim.x * {tpb}) {{")
            self.ind += 1
            self._split_iteration("(appy::i64)__rows[__t]")
            self.ind -= 1
            self.w("}")
        self.mode = "lane"

    # ---- elements grouped by the stripe of the gathered operand they read -------------------------------
    # Blocks of `Spec.block_rows` rows, one wavefront each.  The grouping kernel writes the elements of a block -
    # the 32 bits of the carried operand, the row within the block (10 bits) and the position within the stripe
    # (22 bits) - over the block's own range of positions, stripe after stripe, and where every stripe
    # starts (`__desc`, `parts + 1` numbers per block).  A cell is one stripe of one block.
    @property
    def GROUP_ROWS(self):
        return self.spec.block_rows

    def _group_setup_types(self):
        """Walks the set-up of an iteration and the term of the sum into a buffer that is thrown away:
        the types of the locals settle as they do in the kernels that run the loop row by row.
        Returns (code of the term with `__cv` / `__cx` for the two loads, its type, partial type)."""
        a, g = self.a, self.a.grouping
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        kept, self.lines = self.lines, []
        saved_mode, self.mode = self.mode, "lane"
        self.ex.locals[a.team_split.target.id] = T.WEAK_INT
        self.block(body[:at])
        name = g["name"]
        ty = self.ex.locals.get(name)
        if ty is None:
            raise NameError(f"reduction variable `{name}` has no value before the loop")
        jv = a.team_split.target.id
        x, idx = a.arrays[g["x"]], a.arrays[g["idx"]]
        saved = dict(self.ex.load_subst)
        self.ex.load_subst[f"{g['x']}[{g['idx']}[{jv}]]"] = ("__cx", x.ty)
        if g["carried"]:
            self.ex.load_subst[f"{g['carried']}[{jv}]"] = ("__cv", a.arrays[g["carried"]].ty)
        oc, ot = self.ex.emit(loop_ir.reduction_operand(g["stmt"]))
        self.ex.load_subst = saved
        pty = T.partial_type(ty)
        self.set_local(name, T.promote(ty, ot))
        self.lines, self.mode = kept, saved_mode
        return oc, ot, pty

    def _body_group(self):
        """The grouping kernel.  Per block: the set-up of its rows (and of the first row of the next
        block) gives the rows' ranges, which must follow one another - otherwise the block is refused
        and the flag raised; a first pass over the elements counts them per stripe, a second pass
        writes each element to its place.  The rank of an element within its stripe comes from
        ballots taken in a fixed order, so the layout does not depend on timing."""
        a, g, S, R = self.a, self.a.grouping, self.spec.parts, self.GROUP_ROWS
        var = a.var
        self.ex.locals[var] = T.WEAK_INT
        self.mode = "lane"
        idx_c = cname(g["idx"])
        a.arrays[g["idx"]].loaded = True
        self._group_wide = a.arrays[g["idx"]].ty.size == 8     # 64-bit indices are narrowed as they are loaded
        car_c = f"reinterpret_cast<const int*>({cname(g['carried'])})" if g["carried"] else None
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        U = 4       # vectors of four elements per lane and step
        w = self.w
        w("const int __lid = threadIdx.x & 63;")
        w("const int __wvl = threadIdx.x >> 6;")
        w(f"__shared__ int __lp_all[4][{R + 1}];      // where the rows of the block start; the last entry: where it ends")
        w(f"__shared__ int __hq_all[4][{R + 1}];      // where they end")
        w("int* __lp = __lp_all[__wvl];")
        w("int* __hq = __hq_all[__wvl];")
        if self.spec.skip_long:
            # the sorting kernel of this launch has counted the rows of its classes: they go where the host reads them
            # when it stages the next launch (as the kernel over rows of all classes does)
            w("if (blockIdx.x == 0 && threadIdx.x == 0) {")
            w("    const appy::i64 __others = (__base == 0 ? 0 : (appy::i64)__counts[0]) + (__base == 1 ? 0 : (appy::i64)__counts[1]) "
              "+ (__base == 2 ? 0 : (appy::i64)__counts[2]) + (__base == 3 ? 0 : (appy::i64)__counts[3]);")
            for c in range(4):
                w(f"    __hint[{c + 1}] = (__base == {c}) ? (__hi - __lo) - __others : (appy::i64)__counts[{c}];")
            w("    __hint[0] = 1;")
            w("}")
        w(f"const appy::i64 __nblk = (__hi - __lo + {R - 1}) / {R};")
        w("const int __cmask = (1 << __shiftc) - 1;")
        w("for (appy::i64 __b = (appy::i64)blockIdx.x * 4 + __wvl; __b < __nblk; __b += (appy::i64)gridDim.x * 4) {")
        self.ind += 1
        w(f"const appy::i64 __r0 = __lo + __b * {R};")
        w(f"const int __nr = (int)((__hi - __r0) < {R} ? (__hi - __r0) : {R});")
        w("appy::wave_fence();       // the block before this one has been read out of __lp")
        w("bool __good = true, __long = false;")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{      // and the first row of the next block, if there is one")
        self.ind += 1
        w("const int __r = __k * 64 + __lid;")
        w(f"if (__r <= __nr && __r0 + __r < __hi && (__k < {R // 64} || __lid == 0)) {{")
        self.ind += 1
        w(f"const appy::i64 {cname(var)} = __r0 + __r;")
        self._declare_locals()
        self.block(body[:at])
        lo, hi = self._range_args(a.team_split)
        w(f"const appy::i64 __rlo = {lo};")
        w(f"const appy::i64 __rhi = {hi};")
        w("if (__rlo < 0 || __rhi < __rlo || __rhi > __len) __good = false;")
        w("__lp[__r] = (int)__rlo;")
        w("if (__r < __nr) { __hq[__r] = (int)__rhi; __long = __long || (__rhi - __rlo > __rowmax); }")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("appy::wave_fence();")
        w("// every row ends where the next one starts; the block ends no later than the next one starts")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w("    if (__r < __nr - 1) __good = __good && __lp[__r + 1] == __hq[__r];")
        w("    else if (__r == __nr - 1 && __r0 + __nr < __hi) __good = __good && __lp[__nr] >= __hq[__r];")
        w("}")
        w("__good = __ballot(!__good) == 0ull;")
        if not self.spec.skip_long:
            w("if (__ballot(__long) != 0ull && __lid == 0) __hint[0] = 2;      // rows too long for this treatment: the next launch sorts them")
        w("const int __first = __good ? __lp[0] : 0, __end = __good ? __hq[__nr - 1] : 0;")
        w("appy::wave_fence();")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w(f"    if (__r >= __nr && __r <= {R} && (__k < {R // 64} || __lid == 0)) __lp[__r] = __end;")
        w("}")
        w("appy::wave_fence();")
        w("if (!__good) {")
        w("    // refused: the launch runs the loop row by row instead; the cells of this block stay empty")
        w("    if (__lid == 0) __flag[0] = 1;")
        w(f"    if (__lid <= {S}) __desc[__b * {S + 1} + __lid] = 0;")
        w("    continue;")
        w("}")
        skip = self.spec.skip_long

        def find_row(table, at):
            w(f"int __row = 0, __past = {R};       // the last row that starts at or before {at}")
            w("#pragma unroll")
            w(f"for (int __it = 0; __it < {R.bit_length() - 1}; ++__it) {{")
            w("    const int __mid = (__row + __past) >> 1;")
            w(f"    if ({table}[__mid] <= {at}) __row = __mid; else __past = __mid;")
            w("}")

        def count(k):
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q)")
            w("#pragma unroll")
            w(f"    for (int __s = 0; __s < {S}; ++__s) __cnt[__s] += __popcll(__ballot((__c[{k}][__q] >> __shiftc) == __s));")

        def starts():
            w("__at[0] = __first;")
            w("#pragma unroll")
            w(f"for (int __s = 0; __s < {S}; ++__s) __at[__s + 1] = __at[__s] + __cnt[__s];")
            w("#pragma unroll")
            w(f"for (int __s = 0; __s <= {S}; ++__s) if (__lid == __s) __desc[__b * {S + 1} + __s] = __at[__s];")
            w("int __atv = 0;       // lane s: where the next element of stripe s goes")
            w("#pragma unroll")
            w(f"for (int __s = 0; __s < {S}; ++__s) __atv = __lid == __s ? __at[__s] : __atv;")

        def place_one(kc, kv):
            w(f"const int __cq = __c[{kc}][__q];")
            w("const int __sq = __cq >> __shiftc;          // negative past the end (and for negative indices: such elements are dropped)")
            # the lanes whose element goes to the same stripe, from one ballot per bit of the stripe number (a lane whose
            # bit is set keeps the lanes of the ballot, the others keep the rest); lane s holds where stripe s stands
            w(f"const bool __ok = __sq >= 0 && __sq < {S};")
            w("const unsigned long long __okm = __ballot(__ok);")
            w("unsigned __olo = (unsigned)__okm, __ohi = (unsigned)(__okm >> 32);")
            w("#pragma unroll")
            w(f"for (int __bit = 0; __bit < {(S - 1).bit_length()}; ++__bit) {{")
            w("    const unsigned __e = (unsigned)((__sq << (31 - __bit)) >> 31);       // all ones where the bit is set")
            w("    const unsigned long long __bm = __ballot(__e != 0u);")
            w("    __olo &= ~((unsigned)__bm ^ __e);")
            w("    __ohi &= ~((unsigned)(__bm >> 32) ^ __e);")
            w("}")
            w("const int __pos = __builtin_amdgcn_ds_bpermute(__sq << 2, __atv) "
              "+ (int)__builtin_amdgcn_mbcnt_hi(__ohi, __builtin_amdgcn_mbcnt_lo(__olo, 0u));")
            w("// every lane tells the lane of its stripe how many elements the stripe takes in this step (all of them the same")
            w("// number; a lane that no one tells receives zero; a lane without an element tells what holds for the number it has)")
            w("__atv += __builtin_amdgcn_ds_permute(__sq << 2, __popc(__olo) + __popc(__ohi));")
            w("if (__ok)")
            w("    __ent[__pos] = (long long)(((unsigned long long)(((unsigned)__row << 22) | (unsigned)(__cq & __cmask)) << 32) "
              f"| (unsigned long long)(unsigned)__v[{kv}][__q]);")

        def unrolled(n, fn):
            w("#pragma unroll")
            w(f"for (int __k = 0; __k < {n}; ++__k) {{")
            self.ind += 1
            fn()
            self.ind -= 1
            w("}")

        w(f"int __cnt[{S}], __at[{S + 1}];")
        w("#pragma unroll")
        w(f"for (int __s = 0; __s < {S}; ++__s) __cnt[__s] = 0;")

        def load_indices(k, j0, kk):
            w(f"{{ const int __j = {j0} + {kk} * 256 + __lid * 4;")
            w(f"if (__j + 4 <= __end) __c[{k}] = {self._group_index4(idx_c + ' + __j')};")
            w("else {")
            w("#pragma unroll")
            w(f"    for (int __q = 0; __q < 4; ++__q) __c[{k}][__q] = __j + __q < __end ? {self._group_index1(idx_c + '[__j + __q]')} : -1;")
            w("} }")

        def load_carried(k, j0, kk):
            if car_c:
                w(f"{{ const int __j = {j0} + {kk} * 256 + __lid * 4;")
                w(f"if (__j + 4 <= __end) __v[{k}] = appy::vload<int, 4>({car_c} + __j);")
                w("else {")
                w("#pragma unroll")
                w(f"    for (int __q = 0; __q < 4; ++__q) __v[{k}][__q] = __j + __q < __end ? {car_c}[__j + __q] : 0;")
                w("} }")
            else:
                w(f"__v[{k}] = 0;")

        def place(kc, kv, j0, kk):
            w(f"const int __j = {j0} + {kk} * 256 + __lid * 4;")
            find_row("__lp", "__j")
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q) {")
            self.ind += 1
            w("if (__j + __q < __end) while (__lp[__row + 1] <= __j + __q) ++__row;")
            place_one(kc, kv)
            self.ind -= 1
            w("}")

        if skip:
            # the sorting kernel, which ran before this one, has counted the rows beyond the limit: where there are none,
            # every element is kept and the walk over the arrays as they lie does (the layout is the same either way)
            w("if (__counts[3] == 0) {")
            self.ind += 1
        # (indices of a whole block kept in registers between the two passes - 64 registers, half the wavefronts per
        #  SIMD - made this kernel slower: 455 us against 306 for 2^26 elements)
        w(f"for (int __j0 = __first; __j0 < __end; __j0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}];")
        unrolled(U, lambda: load_indices("__k", "__j0", "__k"))
        unrolled(U, lambda: count("__k"))
        self.ind -= 1
        w("}")
        starts()
        w(f"for (int __j0 = __first; __j0 < __end; __j0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}], __v[{U}];")
        unrolled(U, lambda: (load_indices("__k", "__j0", "__k"), load_carried("__k", "__j0", "__k")))
        unrolled(U, lambda: place("__k", "__k", "__j0", "__k"))
        self.ind -= 1
        w("}")
        if skip:
            self.ind -= 1
            w("} else {")
            self.ind += 1
            self._group_walk_kept(idx_c, car_c, U, find_row, count, starts, place_one, unrolled)
            self.ind -= 1
            w("}")
        self.ind -= 1
        w("}")

    def _group_index4(self, pointer: str) -> str:
        """Four indices of the grouping kernel from `pointer`, as 32-bit numbers (an index that does not fit
        is negative afterwards, and dropped like every negative index)."""
        if not self._group_wide:
            return f"appy::vload<int, 4>({pointer})"
        return f"appy::narrow_indices(appy::vload<long long, 4>({pointer}))"

    def _group_index1(self, value: str) -> str:
        return value if not self._group_wide else f"appy::narrow_index({value})"

    def _group_walk_kept(self, idx_c, car_c, U, find_row, count, starts, place_one, unrolled):
        """The two passes of the grouping kernel over the elements of the rows that are kept (rows
        beyond `__rowmax` elements run in planned parts): the lanes walk the kept elements of the block
        as one sequence; `__kp[r]` is where row r starts in it."""
        R = self.GROUP_ROWS
        w = self.w
        P = R // 64
        w(f"// where every row starts among the elements that are kept (rows beyond the limit hold none): lane l sums rows {P}l .. {P}l + {P - 1}")
        w("int* __kp = __hq;")
        w(f"int __kt[{P}], __mine = 0;")
        w("#pragma unroll")
        w(f"for (int __i = 0; __i < {P}; ++__i) {{")
        w(f"    const int __r = {P} * __lid + __i;")
        w("    const int __n = __r < __nr ? __hq[__r] - __lp[__r] : 0;")
        w("    __kt[__i] = __n > __rowmax ? 0 : __n;")
        w("    __mine += __kt[__i];")
        w("}")
        w("int __incl = __mine;")
        w("#pragma unroll")
        w("for (int __d = 1; __d < 64; __d <<= 1) {")
        w("    const int __o = __shfl_up(__incl, __d, 64);")
        w("    if (__lid >= __d) __incl += __o;")
        w("}")
        w("appy::wave_fence();       // the ends of the rows have been read: their table now holds the starts among the kept")
        w("{")
        w("    int __run = __incl - __mine;")
        w("#pragma unroll")
        w(f"    for (int __i = 0; __i < {P}; ++__i) {{ __kp[{P} * __lid + __i] = __run; __run += __kt[__i]; }}")
        w("}")
        w(f"if (__lid == 63) __kp[{R}] = __incl;")
        w("appy::wave_fence();")
        w(f"const int __kept = __kp[{R}];")

        def positions(k):
            """Row and array positions of the four kept elements __t .. __t + 3 of this lane."""
            w(f"const int __t = __t0 + {k} * 256 + __lid * 4;")
            find_row("__kp", "__t")
            w("int __jq[4];")
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q) {")
            w("    if (__t + __q < __kept) while (__kp[__row + 1] <= __t + __q) ++__row;")
            w("    __jq[__q] = __lp[__row] + (__t + __q - __kp[__row]);")
            w("}")
            w("const bool __run = __t + 4 <= __kept && __jq[3] == __jq[0] + 3;       // four elements in a row of the arrays")

        def load(k, both):
            w("{")
            self.ind += 1
            positions(k)
            w(f"if (__run) __c[{k}] = {self._group_index4(idx_c + ' + __jq[0]')};")
            w("else {")
            w("#pragma unroll")
            w(f"    for (int __q = 0; __q < 4; ++__q) __c[{k}][__q] = __t + __q < __kept ? {self._group_index1(idx_c + '[__jq[__q]]')} : -1;")
            w("}")
            if both:
                if car_c:
                    w(f"if (__run) __v[{k}] = appy::vload<int, 4>({car_c} + __jq[0]);")
                    w("else {")
                    w("#pragma unroll")
                    w(f"    for (int __q = 0; __q < 4; ++__q) __v[{k}][__q] = __t + __q < __kept ? {car_c}[__jq[__q]] : 0;")
                    w("}")
                else:
                    w(f"__v[{k}] = 0;")
            self.ind -= 1
            w("}")

        def place(k):
            w(f"const int __t = __t0 + {k} * 256 + __lid * 4;")
            find_row("__kp", "__t")
            w("#pragma unroll")
            w("for (int __q = 0; __q < 4; ++__q) {")
            self.ind += 1
            w("if (__t + __q < __kept) while (__kp[__row + 1] <= __t + __q) ++__row;")
            place_one(k, k)
            self.ind -= 1
            w("}")

        w(f"for (int __t0 = 0; __t0 < __kept; __t0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}];")
        unrolled(U, lambda: load("__k", False))
        unrolled(U, lambda: count("__k"))
        self.ind -= 1
        w("}")
        starts()
        w(f"for (int __t0 = 0; __t0 < __kept; __t0 += {256 * U}) {{")
        self.ind += 1
        w(f"appy::vec<int, 4>::type __c[{U}], __v[{U}];")
        unrolled(U, lambda: load("__k", True))
        unrolled(U, lambda: place("__k"))
        self.ind -= 1
        w("}")

    def _body_cells(self):
        """The kernel that runs the cells: the term of the sum is evaluated per grouped element (the carried
        operand from the element, the gathered operand from its stripe) and added to the element's row
        in LDS; the sums of a cell's rows go to the scratch table of 4-byte slots per row and stripe."""
        a, g, S, R = self.a, self.a.grouping, self.spec.parts, self.GROUP_ROWS
        self.ex.locals[a.var] = T.WEAK_INT
        self.mode = "lane"
        term, tty, pty = self._group_setup_types()
        if pty.name not in ("float32", "int32", "uint32") and not self.dirty:
            raise Unsupported(f"sums of {pty.name} are not accumulated in LDS")
        x = a.arrays[g["x"]]
        x.loaded = True
        U = 8
        w = self.w
        w("const int __lid = threadIdx.x & 63;")
        w("const int __wvl = threadIdx.x >> 6;")
        w(f"__shared__ {pty.c} __acc_all[4][{R}];        // the sums of the rows of a cell, one cell per wavefront")
        w(f"{pty.c}* __acc = __acc_all[__wvl];")
        w(f"const appy::i64 __nblk = (__hi - __lo + {R - 1}) / {R};")
        w("// workgroup g serves the stripes g mod 8, g mod 8 + 8, ...: workgroups go to the eight XCDs in turn, so every L2")
        w("// holds one stripe of the gathered operand at a time")
        w("const appy::i64 __w0 = (appy::i64)(blockIdx.x >> 3) * 4 + __wvl, __nw = (appy::i64)(gridDim.x >> 3) * 4;")
        w(f"for (int __pass = 0; __pass < {S // 8}; ++__pass) {{")
        self.ind += 1
        w("const int __s = (int)(blockIdx.x & 7) + 8 * __pass;")
        w("const appy::i64 __x0 = (appy::i64)__s << __shiftc;")
        w("for (appy::i64 __b = __w0; __b < __nblk; __b += __nw) {")
        self.ind += 1
        w(f"const int __clo = __desc[__b * {S + 1} + __s], __chi = __desc[__b * {S + 1} + __s + 1];")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) __acc[__k * 64 + __lid] = 0;")
        w("appy::wave_fence();")
        w(f"for (int __j0 = __clo; __j0 < __chi; __j0 += {64 * U}) {{")
        self.ind += 1
        w(f"long long __e[{U}];")
        w(f"{x.elem_c} __xv[{U}];")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        w("    const int __j = __j0 + __k * 64 + __lid;")
        w("    __e[__k] = __j < __chi ? __builtin_nontemporal_load(__ent + __j) : 0ll;")
        w("}")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        w("    const int __j = __j0 + __k * 64 + __lid;")
        w(f"    __xv[__k] = {cname(g['x'])}[__j < __chi ? __x0 + (appy::i64)((unsigned)((unsigned long long)__e[__k] >> 32) & 0x3fffffu) : 0];")
        w("}")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        self.ind += 1
        w("const int __j = __j0 + __k * 64 + __lid;")
        w("if (__j < __chi) {")
        self.ind += 1
        if g["carried"]:
            cty = a.arrays[g["carried"]].ty
            bits = "(int)(unsigned)(unsigned long long)__e[__k]"
            w(f"const {cty.c} __cv = {'__int_as_float(' + bits + ')' if cty.is_float else '(' + cty.c + ')' + bits};")
        w(f"const {x.elem_c} __cx = __xv[__k];")
        w(f"atomicAdd(&__acc[(unsigned)((unsigned long long)__e[__k] >> 54)], {cast(term, tty, pty)});")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("appy::wave_fence();")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64}; ++__k) {{")
        w(f"    const appy::i64 __row = __b * {R} + __k * 64 + __lid;")
        w(f"    if (__row < __hi - __lo) reinterpret_cast<{pty.c}*>(__scratch)[(appy::i64)__s * (__hi - __lo) + __row] = __acc[__k * 64 + __lid];")
        w("}")
        w("appy::wave_fence();")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
