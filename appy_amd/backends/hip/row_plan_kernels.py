"""Kernel bodies for row plans: ``rkeys`` writes the (key, value) pairs the inspector sorts,
``xcells`` runs a finished plan.  A mix-in of :class:`kernelgen.KernelBuilder`."""
from __future__ import annotations

from . import dtypes as T
from .exprs import cast, cname
from .loop_analysis import Unsupported


class RowPlanKernels:
    # ---- row plans: the elements of a sum over a gathered operand, ordered once and kept ----------------
    # A plan orders the elements by cell (a block of 32768 rows x one of eight column ranges of the gathered
    # operand) and, within a cell, by the 128-byte line of the operand they read.  `rkeys` writes one (key,
    # value) pair per element, the library sorts them and works out, tile by tile, where each product goes so
    # that the tile's products lie sorted by row (include/appy_hip.h, "row plans"); `xcells` runs the result.
    PLAN_ROW_BITS = 15

    def _body_rkeys(self):
        """The kernel that writes the pairs.  Per block of 256 rows (one wavefront): the set-up of its rows
        gives the rows' ranges, which must follow one another as those of a CSR matrix do and hold indices
        inside the gathered operand - otherwise the flag is raised and no plan comes of it; then every element
        goes to its own position of the two arrays: the key (block of 32768 rows, line of the operand) and the
        value (bits of the carried operand, row within the block, column within the line)."""
        a, g, R = self.a, self.a.grouping, self.GROUP_ROWS
        var = a.var
        self.ex.locals[var] = T.WEAK_INT
        self.mode = "lane"
        idx_c = cname(g["idx"])
        a.arrays[g["idx"]].loaded = True
        car_c = f"reinterpret_cast<const int*>({cname(g['carried'])})" if g["carried"] else None
        body = a.outer.body
        at = next(k for k, st in enumerate(body) if st is a.team_split)
        U = 4
        w = self.w
        RB = self.PLAN_ROW_BITS
        w("const int __lid = threadIdx.x & 63;")
        w("const int __wvl = threadIdx.x >> 6;")
        w(f"__shared__ int __lp_all[4][{R + 1}];      // where the rows of the block start; the last entry: where it ends")
        w(f"__shared__ int __hq_all[4][{R + 1}];      // where they end")
        w("int* __lp = __lp_all[__wvl];")
        w("int* __hq = __hq_all[__wvl];")
        w(f"const appy::i64 __nblk = (__hi - __lo + {R - 1}) / {R};")
        w("for (appy::i64 __b = (appy::i64)blockIdx.x * 4 + __wvl; __b < __nblk; __b += (appy::i64)gridDim.x * 4) {")
        self.ind += 1
        w(f"const appy::i64 __r0 = __lo + __b * {R};")
        w(f"const int __nr = (int)((__hi - __r0) < {R} ? (__hi - __r0) : {R});")
        w("appy::wave_fence();       // the block before this one has been read out of __lp")
        w("bool __good = true;")
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
        w("if (__r < __nr) __hq[__r] = (int)__rhi;")
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
        w("const int __first = __good ? __lp[0] : 0, __end = __good ? __hq[__nr - 1] : 0;")
        w("appy::wave_fence();")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {R // 64 + 1}; ++__k) {{")
        w("    const int __r = __k * 64 + __lid;")
        w(f"    if (__r >= __nr && __r <= {R} && (__k < {R // 64} || __lid == 0)) __lp[__r] = __end;")
        w("}")
        w("appy::wave_fence();")
        w("if (!__good) {")
        w("    if (__lid == 0) __flag[0] = 1;")
        w("    continue;")
        w("}")
        w("// (how many positions the rows of all blocks cover: when it is every position, no key stays unset and the sort needs a bit less)")
        w("if (__lid == 0) atomicAdd(reinterpret_cast<unsigned long long*>(__flag) + 1, (unsigned long long)(__end - __first));")
        w(f"const unsigned __rel0 = (unsigned)(__b * {R});       // first row of the block, counted from the start of the range")
        w("bool __inside = true;")
        w(f"for (int __j0 = __first; __j0 < __end; __j0 += {256 * U}) {{")
        self.ind += 1
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {U}; ++__k) {{")
        self.ind += 1
        w("const int __j = __j0 + __k * 256 + __lid * 4;")
        w("if (__j >= __end) continue;")
        ic = a.arrays[g["idx"]].elem_c           # int, or long long: narrowed once it is known to lie inside the operand
        w(f"appy::vec<{ic}, 4>::type __c;")
        w("appy::vec<int, 4>::type __v;")
        w(f"if (__j + 4 <= __end) __c = appy::vload<{ic}, 4>({idx_c} + __j);")
        w("else {")
        w("#pragma unroll")
        w(f"    for (int __q = 0; __q < 4; ++__q) __c[__q] = __j + __q < __end ? {idx_c}[__j + __q] : 0;")
        w("}")
        if car_c:
            w(f"if (__j + 4 <= __end) __v = appy::vload<int, 4>({car_c} + __j);")
            w("else {")
            w("#pragma unroll")
            w(f"    for (int __q = 0; __q < 4; ++__q) __v[__q] = __j + __q < __end ? {car_c}[__j + __q] : 0;")
            w("}")
        else:
            w("__v = 0;")
        w(f"int __row = 0, __past = {R};       // the last row that starts at or before __j")
        w("#pragma unroll")
        w(f"for (int __it = 0; __it < {R.bit_length() - 1}; ++__it) {{")
        w("    const int __mid = (__row + __past) >> 1;")
        w("    if (__lp[__mid] <= __j) __row = __mid; else __past = __mid;")
        w("}")
        # (four keys and four values leave as vectors where the lane holds four elements inside the operand: one store
        #  of 16 bytes and two instead of eight single ones)
        w("appy::vec<unsigned, 4>::type __kq;")
        w("appy::vec<unsigned long long, 4>::type __vq;")
        w("bool __all = __j + 4 <= __end;")
        w("#pragma unroll")
        w("for (int __q = 0; __q < 4; ++__q) {")
        w("    if (__j + __q < __end) while (__lp[__row + 1] <= __j + __q) ++__row;")
        w(f"    const {ic} __cq = __c[__q];")
        w("    const bool __in = __cq >= 0 && __cq < __nx;")
        w("    if (__j + __q < __end && !__in) __inside = false;")
        w("    __all = __all && __in;")
        w("    const unsigned __rel = __rel0 + (unsigned)__row;")
        w(f"    __kq[__q] = ((__rel >> {RB}) << __lbits) | ((unsigned)__cq >> 5);")
        w(f"    __vq[__q] = (unsigned long long)(unsigned)__v[__q] | ((unsigned long long)((__rel & {(1 << RB) - 1}u) "
          f"| (((unsigned)__cq & 31u) << {RB})) << 32);")
        w("}")
        w("if (__all) {")
        w("    appy::vstore<unsigned, 4>(__keys + __j, __kq);")
        w("    appy::vstore<unsigned long long, 4>(__vals + __j, __vq);")
        w("} else {")
        w("#pragma unroll")
        w("    for (int __q = 0; __q < 4; ++__q) {")
        w(f"        const {ic} __cq = __c[__q];")
        w("        if (__j + __q < __end && __cq >= 0 && __cq < __nx) { __keys[__j + __q] = __kq[__q]; __vals[__j + __q] = __vq[__q]; }")
        w("    }")
        w("}")
        self.ind -= 1
        w("}")
        self.ind -= 1
        w("}")
        w("if (__ballot(!__inside) != 0ull && __lid == 0) __flag[0] = 1;      // an index outside the gathered operand: no plan")
        self.ind -= 1
        w("}")

    def _body_xcells(self):
        """The kernel that runs a row plan: workgroups of 1024 lanes (one per CU: their LDS allows no more), the
        cells of column range g on the workgroups g mod 8 (one XCD and its L2 per range); a workgroup walks the
        tiles of its cells as one sequence, so that the loads of a cell's first tiles travel while the cell before
        it is finished, and puts out the sums of a cell when its last tile is through.  Tile by tile: the lanes gather the
        operand in the order of the plan (adjacent lanes read the same lines), put the value of each term into
        its slot in LDS, and after a barrier add the slots to the sums of the cell's rows, which are in LDS
        too - first the rows with one slot, a lane per row, then the rows with a run of slots, a lane per run,
        in slot order.  A row is touched by one lane per tile and tiles are separated by barriers: the sums do
        not depend on timing.  The sums of a cell go to the scratch table of 4-byte slots per row and range.

        A wavefront instruction takes four cycles on a SIMD and only four wavefronts share one, so the loop is
        written for few instructions: every load is a per-tile base held in scalar registers plus a lane
        offset that never changes, nothing is loaded under a branch (a tile that does not exist is read at one
        position for every lane and never used), the starts of a cell come through the scalar cache, and the header
        of a tile becomes a scalar one stage after it was asked for."""
        a, g = self.a, self.a.grouping
        U = self.spec.unroll
        TILE = 1024 * U
        H = U // 2
        SEG = TILE // 2 + 4          # words of the row stream from one tile of a cell to the next
        RB = self.PLAN_ROW_BITS
        ROWS = 1 << RB
        self.ex.locals[a.var] = T.WEAK_INT
        self.mode = "lane"
        term, tty, pty = self._group_setup_types()
        if pty.name not in ("float32", "int32", "uint32") and not self.dirty:
            raise Unsupported(f"sums of {pty.name} are not accumulated in LDS")
        x = a.arrays[g["x"]]
        x.loaded = True
        xc = cname(g["x"])
        w = self.w
        P = pty.c

        def value(e, xv):
            """Code of the term for element word `e` and gathered value `xv`."""
            pre = ""
            if g["carried"]:
                cty = a.arrays[g["carried"]].ty
                bits = f"(int)(unsigned)({e})"
                pre = f"const {cty.c} __cv = {'__int_as_float(' + bits + ')' if cty.is_float else '(' + cty.c + ')' + bits}; "
            return f"{{ {pre}const {x.elem_c} __cx = {xv}; __val = {cast(term, tty, pty)}; }}"

        w("const unsigned __tid = threadIdx.x;")
        w(f"__shared__ {P} __sum[{ROWS}];        // the sums of the rows of the cell")
        w(f"__shared__ __attribute__((aligned(8))) {P} __prod[{TILE}];       // the terms of a tile, sorted by row")
        w("const appy::i64 __n = __hi - __lo;")
        w("const unsigned __cmask = (1u << __colbits) - 1u;")
        w("const unsigned __xlast = (unsigned)(__nx - 1);")
        w("const char* __xb = reinterpret_cast<const char*>(" + xc + ");")
        w("// A cell may be shared by __split workgroups, each with a run of its tiles and a slot of its own for the sums: a")
        w("// run is numbered (block * __split + part) * 8 + range.  The workgroup takes the runs that the entries blockIdx.x,")
        w("// blockIdx.x + gridDim.x, ... of __order name (dealt out on the host by size; the grid is a multiple of eight")
        w("// workgroups and all runs of a workgroup read the same range) and walks their tiles as one sequence, so that")
        w("// the loads of a run's first tiles travel while the run before it is finished.")
        w("const unsigned __nrun = (unsigned)(__ncell * __split), __spl = (unsigned)__split;")
        w("const unsigned __g = blockIdx.x & 7u;")
        w("const unsigned __x0 = __g * (unsigned)__gwidth;")
        w("#pragma unroll")
        w(f"for (int __k = 0; __k < {ROWS // 1024}; ++__k) __sum[__k * 1024 + __tid] = 0;")
        w(f"unsigned long long __e0[{U}], __e1[{U}], __e2[{U}];")
        w(f"{x.elem_c} __xv[{U}], __x1[{U}];")
        w(f"unsigned __r0[{H}], __r1[{H}];")
        w("unsigned __da0, __db0, __da1, __db1;")
        w("unsigned __h0, __h1, __hv2;        // headers of the tiles in flight (the newest as it was loaded, in a vector register)")
        w("// the tile the next load fetches: run, tile within the run; of the run: its tiles, where its elements and its row")
        w("// stream start, the elements from there to the end of the cell")
        w("unsigned __vi = blockIdx.x, __tt = 0, __nt = 0;")
        w("unsigned __vc = __vi < __norder ? __order[__vi] : 0xffffffffu;        // (no run: a number beyond them all)")
        w("appy::i64 __eb = 0, __sb = 0;      // (in bytes from the start of the elements and of the row stream)")
        w("const char* __entb = reinterpret_cast<const char*>(__ent);")
        w("const char* __rsb = reinterpret_cast<const char*>(__rstream);")
        w("appy::i64 __left = 0;")
        w("// of the tiles in flight (0: the one that is added up, 1: the one whose gathers travel, 2: the one just requested):")
        w("// whether it exists, its elements, whether it ends its run, the run, its part of the row stream")
        w("bool __in0, __in1, __in2, __end0, __end1, __end2, __any0, __any1, __any2;")
        w("unsigned __cnt0, __cnt1, __cnt2, __run0, __run1, __run2;")
        w("appy::i64 __ps0, __ps1, __ps2;")

        def enter_run():
            """Where the run __vc lies (when there is such a run)."""
            w("if (__vc < __nrun) {")
            w("    const unsigned __b = (__vc >> 3) / __spl, __part = (__vc >> 3) % __spl;")
            w("    const appy::i64 __cell = (appy::i64)__b * 8 + __g;")
            w("    const unsigned __nta = __tbase[__cell + 1] - __tbase[__cell];")
            w("    const unsigned __tlo = __part * __nta / __spl;        // (at most 32 parts, and tiles of thousands of elements)")
            w("    __nt = (__part + 1) * __nta / __spl - __tlo;")
            w(f"    const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * {TILE};")
            w("    __left = (appy::i64)__cstart[__cell + 1] - __cs;")
            w("    __eb = __cs * 8;")
            w("    __sb = ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)) * 4;")
            w("} else {")
            w("    __nt = 0;")
            w("}")

        # (a tile that does not exist - past the last run, or the one turn of a run without tiles - is read all the
        #  same: one position for every lane, so that it costs one request per instruction, and never used)
        def load_tile(dst):
            """Requests the header and the elements of the next tile of the sequence into stage 2, and steps on.
            (The header is asked for first and as a vector load, and turned into a scalar only when the tile moves on
            to stage 1: a wait for it then covers no load younger than it, and none that misses.)"""
            w("{")
            w("  __any2 = __vc < __nrun; __in2 = __any2 && __tt < __nt; __end2 = __tt + 1 >= __nt; __run2 = __vc;")
            w(f"  const char* __p = __entb + appy::uniform_i64(__in2 ? __eb + (appy::i64)__tt * {TILE * 8} : 0);")
            w(f"  __ps2 = appy::uniform_i64(__in2 ? __sb + (appy::i64)__tt * {SEG * 4} : 0);")
            w("  __hv2 = *reinterpret_cast<const unsigned*>(__rsb + __ps2 + appy::lane_offset(0u));")
            w(f"  const appy::i64 __l = __left - (appy::i64)__tt * {TILE};")
            w(f"  __cnt2 = __in2 ? (unsigned)(__l < {TILE} ? __l : {TILE}) : 0u;")
            w("#pragma unroll")
            w(f"  for (int __u = 0; __u < {U}; ++__u)")
            w(f"      {dst}[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + appy::lane_offset(__in2 ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));")
            w("  if (__any2) {")
            w("      if (!__end2) ++__tt;")
            w("      else {")
            w("          __vi += gridDim.x; __vc = __vi < __norder ? __order[__vi] : 0xffffffffu; __tt = 0;")
            self.ind += 3
            enter_run()
            self.ind -= 3
            w("      }")
            w("  }")
            w("}")

        def load_rows(dst, da, db, hdr, inn, ps):
            """Row numbers of the slots this lane adds up, and the first run of slots it may have to walk."""
            w("{")
            w("#pragma unroll")
            w(f"  for (int __u = 0; __u < {H}; ++__u)")
            w(f"      {dst}[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(__rsb + {ps} + appy::lane_offset({inn} ? (unsigned)((1 + __u * 1024 + __tid) * 4) : 0u)));")
            w(f"  const unsigned __runs = ({hdr} >> 16);")
            w(f"  const char* __q = __rsb + ({ps} + ({inn} ? (appy::i64)(1 + ((({hdr} & 0xffffu) + 1) >> 1)) * 4 : 0));     // (the header of a tile that does not exist may hold anything)")
            w(f"  const unsigned __at = appy::lane_offset({inn} && __tid < __runs ? __tid * 4 : 0u);        // (lanes without a run: one position)")
            w(f"  {da} = *reinterpret_cast<const unsigned*>(__q + __at);")
            w(f"  {db} = *reinterpret_cast<const unsigned*>(__q + __at + 4); }}")

        def gather(dst, src, inn, first, last):
            w("{")
            w("#pragma unroll")
            w(f"  for (int __u = {first}; __u < {last}; ++__u) {{")
            w(f"    unsigned __c = __x0 + ((unsigned)({src}[__u] >> 32) & __cmask);")
            w("    __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)")
            w(f"    {dst}[__u] = *reinterpret_cast<const {x.elem_c}*>(__xb + appy::lane_offset({inn} ? (unsigned)(__c << 2) : 0u));")
            w("  } }")

        def shift(frm, to):
            w(f"__in{to} = __in{frm}; __end{to} = __end{frm}; __any{to} = __any{frm}; __cnt{to} = __cnt{frm}; "
              f"__run{to} = __run{frm}; __ps{to} = __ps{frm};")

        def add_run(d, d1):
            w(f"{{ const int __row = (int)({d} & {ROWS - 1}u), __from = (int)({d} >> {RB}), __to = (int)({d1} >> {RB});")
            w(f"  {P} __acc = __sum[__row];")
            w("  for (int __k = __from; __k < __to; __k += 4) {")
            w(f"      const {P} __p0 = __prod[__k], __p1 = __k + 1 < __to ? __prod[__k + 1] : 0, "
              "__p2 = __k + 2 < __to ? __prod[__k + 2] : 0, __p3 = __k + 3 < __to ? __prod[__k + 3] : 0;")
            w("      __acc += __p0;")
            w("      if (__k + 1 < __to) __acc += __p1;")
            w("      if (__k + 2 < __to) __acc += __p2;")
            w("      if (__k + 3 < __to) __acc += __p3;")
            w("  }")
            w("  __sum[__row] = __acc; }")

        enter_run()
        load_tile("__e0")
        w("__h0 = __builtin_amdgcn_readfirstlane(__hv2);")
        shift(2, 0)
        load_tile("__e1")
        w("__h1 = __builtin_amdgcn_readfirstlane(__hv2);")
        shift(2, 1)
        load_rows("__r0", "__da0", "__db0", "__h0", "__in0", "__ps0")
        gather("__xv", "__e0", "__in0", 0, U)
        w("__syncthreads();")
        w("while (__any0) {")
        self.ind += 1
        w("const unsigned __ns = __in0 ? __h0 & 0xffffu : 0u, __nm = __in0 ? __h0 >> 16 : 0u;")
        # Where the loads of the next tiles are asked for was settled with cycle counters at the boundaries of the phases: a
        # wave that asks for a load waits until the texture addresser takes it, and with every load ahead of the first
        # barrier all waves stood in that queue together (7000 of 11300 cycles per tile) while LDS was idle, and then
        # added up together while the addresser was idle.  So the element stream of the tile after the next goes first (it
        # comes from HBM), the row numbers follow the scatter, and the gathers are asked for in two halves between the
        # phases that add up: waves that have been served go on adding while the others queue.
        load_tile("__e2")
        w(f"if (__cnt0 == {TILE}u) {{")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {U}; ++__u) {{")
        w(f"        {P} __val;")
        w("        " + value("__e0[__u]", "__xv[__u]"))
        w("        __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;")
        w("    }")
        w("} else {")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {U}; ++__u) {{")
        w(f"        {P} __val;")
        w("        " + value("__e0[__u]", "__xv[__u]"))
        w("        if (__u * 1024 + __tid < __cnt0) __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;")
        w("    }")
        w("}")
        load_rows("__r1", "__da1", "__db1", "__h1", "__in1", "__ps1")
        w("__syncthreads();")
        w("{")
        w(f"    {P} __sa[{H}], __sb_[{H}];")
        w(f"    appy::vec<{P}, 2>::type __pp[{H}];")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {H}; ++__u) {{")
        w(f"        __pp[__u] = *reinterpret_cast<const appy::vec<{P}, 2>::type*>(&__prod[2 * (__u * 1024 + __tid)]);")
        w("        __sa[__u] = __sum[__r0[__u] & 0x7fffu]; __sb_[__u] = __sum[(__r0[__u] >> 16) & 0x7fffu];")
        w("    }")
        w("#pragma unroll")
        w(f"    for (int __u = 0; __u < {H}; ++__u) {{")
        w("        const unsigned __s = 2 * (__u * 1024 + __tid);")
        w("        if (__s < __ns) __sum[__r0[__u] & 0x7fffu] = __sa[__u] + __pp[__u][0];")
        w("        if (__s + 1 < __ns) __sum[(__r0[__u] >> 16) & 0x7fffu] = __sb_[__u] + __pp[__u][1];")
        w("    }")
        w("}")
        gather("__x1", "__e1", "__in1", 0, H)
        w("if (__nm > 0) {")
        self.ind += 1
        w("if (__tid < __nm) {")
        self.ind += 1
        add_run("__da0", "__db0")
        self.ind -= 1
        w("}")
        w("if (__nm > 1024) {")
        w("    const unsigned* __runs = reinterpret_cast<const unsigned*>(__rsb + __ps0) + 1 + ((__ns + 1) >> 1);")
        w("    for (unsigned __m = __tid + 1024; __m < __nm; __m += 1024) {")
        w("        const unsigned __d = __runs[__m], __d1 = __runs[__m + 1];")
        self.ind += 2
        add_run("__d", "__d1")
        self.ind -= 2
        w("    }")
        w("}")
        self.ind -= 1
        w("}")
        gather("__x1", "__e1", "__in1", H, U)
        w("__syncthreads();")
        w("if (__end0) {")
        self.ind += 1
        w("// the run is through: its sums go out and start again at zero (every lane clears what it has read itself; the next")
        w("// tile's terms are added after the barrier that follows their scatter)")
        w("const unsigned __b = (__run0 >> 3) / __spl, __part = (__run0 >> 3) % __spl;")
        w(f"{P}* __out = reinterpret_cast<{P}*>(__scratch) + ((appy::i64)__part * 8 + __g) * __n + (appy::i64)__b * {ROWS};")
        w(f"if (((appy::i64)__b + 1) * {ROWS} <= __n) {{")
        w("#pragma unroll")
        w(f"    for (int __k = 0; __k < {ROWS // 1024}; ++__k) {{ __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid]; __sum[__k * 1024 + __tid] = 0; }}")
        w("} else {")
        w(f"    for (int __k = 0; __k < {ROWS // 1024}; ++__k) {{")
        w(f"        if ((appy::i64)__b * {ROWS} + __k * 1024 + __tid < __n) __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid];")
        w("        __sum[__k * 1024 + __tid] = 0;")
        w("    }")
        w("}")
        self.ind -= 1
        w("}")
        w("#pragma unroll")
        w(f"for (int __u = 0; __u < {U}; ++__u) {{ __e0[__u] = __e1[__u]; __e1[__u] = __e2[__u]; __xv[__u] = __x1[__u]; }}")
        w("#pragma unroll")
        w(f"for (int __u = 0; __u < {H}; ++__u) __r0[__u] = __r1[__u];")
        w("__h0 = __h1; __h1 = __builtin_amdgcn_readfirstlane(__hv2); __da0 = __da1; __db0 = __db1;")
        shift(1, 0)
        shift(2, 1)
        self.ind -= 1
        w("}")
