#!/usr/bin/env python3
"""Writes prefill_mfma_loop.inc: the tile loop of prefill_asm_kernel as one inline-assembly block per head size
(128, 64, 32), element type (bf16, fp16) and variant (without / with lower bounds).

Why assembly: with one wave per SIMD nothing hides latency except the wave's own instruction order, and a
wave issues one instruction per 4 cycles (a matrix product takes two issue slots, an exponential two).  At
head_dim 128 a 32-key subtile is 32 products = 1024 cycles = 256 issue slots, and the softmax arithmetic,
operand reads and tile loads around them need about 230: the loop only runs near the matrix unit's rate if next
to nothing else is issued and the other instructions are spread evenly between the products.  At head_dim 64
the subtile has 16 products and nearly the same softmax arithmetic (it goes with keys x rows, not with the head
size): about 200 slots of other instructions against 512 cycles of products, so the issue rate bounds that
loop and every instruction saved counts in full.  This script fixes the
register assignment, places every instruction, derives the `s_waitcnt lgkmcnt` values from the order of the
LDS reads and checks the distances the hardware does not interlock (matrix result -> vector read,
transcendental -> vector read, vector write -> lane swap).

The loop runs every tile of 64 keys of the workgroup, for every wave, four tiles (one turn of the LDS ring)
per iteration.  Per tile t: publish tile t+1 (wait for this wave's loads, zero rows that do not exist,
barrier), issue the loads of tile t+3, and per 32-key subtile g: exponentials of S^T(g) and the O^T products,
with the S^T products and row maxima of subtile g+1 between them.  Keys a row must not see (causal mask,
context end) are set to -inf in a block of compare/select pairs that is skipped for subtiles no row of the
wave needs it for.  A wave whose rows end before the workgroup's last tile keeps going with everything
masked (its probabilities are exact zeros), and loads past the last tile fetch tile 0 again, so that every
wave executes the same barriers and the same number of loads per tile.

Register map (per lane; the kernel pins its variables to the same registers; KS = head_dim / 16 k-steps of
S^T, DT = head_dim / 32 d tiles of O^T; the ranges are those of head_dim 128, head_dim 64 uses the first half
of each, head_dim 32 the first quarter):
  a[0:127]    O^T accumulators  o[c][dt]   at 16*(DT*c + dt)
  a[128:191]  Q^T operands      q[c][ks]   at 128 + 4*(KS*c + ks)
  a[192:223]  K operands        ka[ks]     at 192 + 4*ks
  a[224:239]  V^T operands of the first k-step (d tile dt at 224 + 4*dt), a[240:255] of the second
  v[0:63]     S^T: buffer b, column tile c at 16*(2b+c); a tile starts with its first subtile in buffer 0
  v[64:79]    P^T operand words pp[c][j] at 64 + 8c + j
  v[80:87]    exponentials in flight, v[88:91] four table entries, v92 table address, v[93:96] maxima
              (v95 also a row's last visible key relative to the subtile), v[97:98] pair sums, v99 scratch
  v[100:111]  LDS addresses of stages 2 and 3 (the operands hold those of stages 0 and 1)
  v[112:115]  zeros, v116 -inf
  v[118:149]  minus the rows' reference maxima, one 16-register tile per column tile (the accumulator input of
              the first S^T product)
  s[40:63]    scalars of the tile loads, the calls, the masks and the rescale checks

Usage: python3 gen_prefill_loop.py [output file]   (default: prefill_mfma_loop.inc beside this script)
"""
import os
import sys

NC, NSTAGE = 2, 4


def configure(head_dim):
    """The shape constants of a head size (128, 64 or 32; 16-bit elements)."""
    global D, KS, DT, RB, TENSOR, STAGE, M_A, M_B, GAPS, SYNC_GAP, NG, MAX_GAP
    D = head_dim
    KS, DT = D // 16, D // 32   # k-steps of S^T = K . Q^T, 32-wide d tiles of O^T
    RB = 2 * D                   # bytes of a K / V row
    TENSOR = 64 * RB             # one tensor's tile of 64 keys
    STAGE = 2 * TENSOR           # K tile + V tile
    M_A, M_B = NC * KS, NC * DT  # products of S^T, and of one k-step of O^T, per subtile
    GAPS = M_A + 2 * M_B + 1     # places for other instructions around the products of a subtile
    SYNC_GAP = M_A               # where tile t+1 is published in a tile's first subtile
    NG = RB // 64                # direct loads per wave, tile and tensor (a tensor's tile is 64 * RB bytes, a wave load 1 KiB, 4 waves)
    MAX_GAP = {128: 21, 64: 11, 32: 5}[D]  # first gap of the row maxima (far enough behind the last S^T product)


configure(128)


def areg(base, n):
    return f"a[{base}:{base + n - 1}]"


def vreg(base, n):
    return f"v[{base}:{base + n - 1}]"


def O(c, dt):
    return areg(16 * (DT * c + dt), 16)


def Q(c, ks):
    return areg(128 + 4 * (KS * c + ks), 4)


def KA(ks):
    return 192 + 4 * ks


def VA(step, dt):
    return 224 + 16 * step + 4 * dt


def S(buf, c):
    return 16 * (2 * buf + c)


def PP(c, j):
    return 64 + 8 * c + j


def CT(c):
    return 118 + 16 * c


LO = False  # the variant being generated also applies lower bounds (sliding window, per-row first keys)
STUBS = []  # out-of-line code of the loop being generated: the common path of every check falls through


class Ins:
    """One instruction (or an inseparable group written as several lines)."""

    def __init__(self, text, units=1, kind="valu", reads=(), writes=(), need=(), issue=None, n=1):
        self.text, self.units, self.kind = text, units, kind
        self.reads, self.writes = tuple(reads), tuple(writes)  # VGPR numbers ("v12") it reads / writes
        self.need = tuple(need)   # LDS register groups that must have arrived
        self.issue = issue        # LDS register group this read fills
        self.n = n                # instructions in the group (wait states it provides)


class Op:
    def __init__(self, ins, earliest=0, latest=None):
        self.ins = ins if isinstance(ins, list) else [ins]
        self.earliest, self.latest = earliest, GAPS - 1 if latest is None else latest
        self.units = sum(i.units for i in self.ins)


class Types:
    def __init__(self, name):
        self.name = name
        if name == "bf16":
            self.mfma = "v_mfma_f32_32x32x16_bf16"
            self.dot2 = "v_dot2_f32_bf16"
            self.ones = "0x3f803f80"
        else:
            self.mfma = "v_mfma_f32_32x32x16_f16"
            self.dot2 = "v_dot2_f32_f16"
            self.ones = "0x3c003c00"

    def pack(self, dst, a, b):
        # (gfx950 converts a pair to either 16-bit type in one instruction, round to nearest even)
        op = "v_cvt_pk_bf16_f32" if self.name == "bf16" else "v_cvt_pk_f16_f32"
        return [Ins(f"{op} v{dst}, v{a}, v{b}", reads=(f"v{a}", f"v{b}"), writes=(f"v{dst}",))]


def k_addr(stage, ks):
    """(register, immediate) of the K operand read base of a ring stage."""
    reg = f"%[kad{ks}]" if stage < 2 else f"v{100 + ks}"
    return reg, (stage & 1) * STAGE


def v_addr(stage, dt):
    reg = f"%[vad{dt}]" if stage < 2 else f"v{108 + dt}"
    return reg, (stage & 1) * STAGE


def subtile_ops(ty, j, kt):
    """Products and the other instructions of subtile kt of the tile at unroll position j (ring stage j)."""
    cb, nb = kt & 1, 1 - (kt & 1)
    mf = []
    for ks in range(KS):
        for c in range(NC):
            s = S(nb, c)
            # The first product of a column tile accumulates onto minus the row's reference maximum (the same
            # value in all 16 registers of a lane), and Q^T arrives scaled by softmax scale * log2(e): S^T comes
            # out as the argument of the exponential, and no instruction per value is spent on forming it.
            src_c = vreg(CT(c), 16) if ks == 0 else vreg(s, 16)
            mf.append(Ins(f"{ty.mfma} {vreg(s, 16)}, {areg(KA(ks), 4)}, {Q(c, ks)}, {src_c}", units=2, kind="mfma",
                          reads=[f"v{CT(c) + i}" for i in range(16)] if ks == 0 else (),
                          writes=[f"v{s + i}" for i in range(16)], need=(f"ka{ks}",)))
    for step in range(2):
        for dt in range(DT):
            for c in range(NC):
                p = PP(c, 4 * step)
                mf.append(Ins(f"{ty.mfma} {O(c, dt)}, {areg(VA(step, dt), 4)}, {vreg(p, 4)}, {O(c, dt)}", units=2,
                              kind="mfma", reads=[f"v{p + i}" for i in range(4)], need=(f"va{step}_{dt}",)))
    streams = {}

    # ---- rescale check (start of the subtile) ----
    # (the two compares sit behind the maxima of the previous subtile, so their results are long there)
    chk = [Ins("s_or_b64 vcc, s[60:61], s[62:63]", kind="salu"),
           Ins(f"s_cbranch_vccnz .Lpf_rescale_{j}{kt}_%=\n.Lpf_rescaled_{j}{kt}_%=:", kind="salu", n=1)]
    STUBS.append([f".Lpf_rescale_{j}{kt}_%=:", "s_call_b64 s[50:51], .Lpf_rescale_%=", f"s_branch .Lpf_rescaled_{j}{kt}_%="])
    streams["chk"] = [Op(chk, 0, 0)]

    # ---- LDS operand reads ----
    lds = []

    # One operand read per gap, each pinned to its own gap: a burst of LDS reads holds up the wave's only instruction
    # stream while the four waves of the workgroup, in step behind the barrier, queue at the LDS together
    # (measured: +2 % on the whole kernel against reads placed as early as their deadlines allow).
    def v_reads(step, sub_stage, sub_kt, first):
        for dt in range(DT):
            reg, imm = v_addr(sub_stage, dt)
            base = imm + (32 * sub_kt + 16 * step) * RB
            gap = first + 2 * dt
            lds.append(Op(Ins(f"ds_read_b64_tr_b16 {areg(VA(step, dt), 2)}, {reg} offset:{base}", kind="lds"), gap, gap))
            lds.append(Op(Ins(f"ds_read_b64_tr_b16 {areg(VA(step, dt) + 2, 2)}, {reg} offset:{base + 8 * RB}", kind="lds",
                              issue=f"va{step}_{dt}"), gap + 1, gap + 1))

    v_reads(0, j, kt, 0)       # first k-step of this subtile: consumed from product M_A on
    v_reads(1, j, kt, 2 * DT)  # second k-step: consumed from product M_A + M_B on
    if kt == 0:
        # tile j+1 becomes visible: this wave's loads of it have landed, then every wave's
        # (a tile in [splo, splo + spspan) has rows past the context end or in absent blocks: the wave clears the
        # rows it loaded itself; unsigned compare of the distance covers both ends)
        lds.append(Op(Ins(f"s_waitcnt vmcnt({2 * NG})\n\ts_sub_u32 s56, %[sP], %[splo]\n\ts_cmp_lt_u32 s56, %[spspan]\n"
                          f"\ts_cbranch_scc1 .Lpf_fix_{j}_%=\n.Lpf_fixed_{j}_%=:\n"
                          "\ts_add_u32 %[sP], %[sP], 1\n\ts_barrier",
                          kind="sync", units=6, n=6), SYNC_GAP, SYNC_GAP))
        STUBS.append([f".Lpf_fix_{j}_%=:", "s_call_b64 s[50:51], .Lpf_fixup_%=", f"s_branch .Lpf_fixed_{j}_%="])
    # K operands of subtile g+2 = subtile kt of the next tile (stage j+1)
    nstage = (j + 1) % NSTAGE
    for ks in range(KS):
        reg, imm = k_addr(nstage, ks)
        lds.append(Op(Ins(f"ds_read_b128 {areg(KA(ks), 4)}, {reg} offset:{imm + kt * 32 * RB}", kind="lds", issue=f"ka{ks}"),
                      SYNC_GAP + 1 + ks, SYNC_GAP + 1 + ks))
    streams["lds"] = lds

    # ---- exponentials: piece n covers S^T values 2j', 2j'+1 of column tile c (n = 2j' + c) ----
    pcs = []

    def half_a(n):
        c, jj = n & 1, n >> 1
        s0 = S(cb, c) + 2 * jj
        ta, tb = 80 + 2 * (n % 4), 81 + 2 * (n % 4)
        return [Ins(f"v_exp_f32_e32 v{ta}, v{s0}", units=2, kind="trans", reads=(f"v{s0}",), writes=(f"v{ta}",)),
                Ins(f"v_exp_f32_e32 v{tb}, v{s0 + 1}", units=2, kind="trans", reads=(f"v{s0 + 1}",), writes=(f"v{tb}",))]

    # The row sums are plain fp32 additions: v_dot2 on the packed words would be one instruction instead of
    # two, but it does not run beside the matrix unit (measured: a product followed by two of them takes 58
    # cycles instead of 32).  The pair is added first and joins the running sum one piece later, so no addition waits for the one before it.
    def half_b(n):
        c, jj = n & 1, n >> 1
        ta, tb = 80 + 2 * (n % 4), 81 + 2 * (n % 4)
        p = PP(c, jj)
        pr = 97 + (n & 1)  # the pair's sum (v97 / v98: also the rescale call's scratch, which runs when neither is live)
        out = [Ins(f"v_add_f32_e32 v{pr}, v{ta}, v{tb}", reads=(f"v{ta}", f"v{tb}"), writes=(f"v{pr}",))] + ty.pack(p, ta, tb)
        if n >= 1:
            pc, ppr = (n - 1) & 1, 97 + ((n - 1) & 1)
            out.append(Ins(f"v_add_f32_e32 %[l{pc}], %[l{pc}], v{ppr}", reads=(f"v{ppr}",)))
        if n == 15:
            out.append(Ins(f"v_add_f32_e32 %[l{c}], %[l{c}], v{pr}", reads=(f"v{pr}",)))
        return out

    def deadline(n):  # a whole gap before the product that reads the word
        return M_A - 2 if n < 8 else M_A + M_B - 2

    # (every instruction is placed on its own; the order keeps the four instructions of the next piece between an
    # exponential and the conversion that reads it)
    for n in range(16):
        pcs += [Op(ins, 0, deadline(n)) for ins in half_a(n)]
        if n >= 1:
            pcs += [Op(ins, 0, deadline(n - 1)) for ins in half_b(n - 1)]
    pcs += [Op(ins, 0, deadline(15)) for ins in half_b(15)]
    streams["pcs"] = pcs

    # ---- row maxima of the next subtile's S^T (complete once product 15 has written it) ----
    mx = []
    m = [93, 94]   # running maxima
    w = [95, 96]   # copies for the half-wave exchange
    # keys a row must not see.  srem = maskfrom - 64*t in tile t; the S^T formed in subtile kt starts at key
    # 64*t + 32*(kt+1) and needs the mask if it reaches past maskfrom: srem < 32*(kt+2).  Value i of a lane is key
    # 8*(i/4) + i%4 of the subtile (+ 4*half, folded into lim), visible up to lim - first key of the subtile.
    # With lower bounds (LO): slo = (first key the wave's last row sees) - 64*t; the same S^T needs the mask too if
    # it starts below that key: slo > 32*(kt+1); a value is then also masked below lo - first key of the subtile.
    blk = [f".Lpf_mask_{j}{kt}_%=:"]
    for c in range(NC):
        s = S(nb, c)
        blk += [f"v_subrev_u32_e32 v95, %[maskfrom], %[lim{c}]", "v_add_u32_e32 v95, %[srem], v95",
                f"v_subrev_u32_e32 v95, {32 * (kt + 1)}, v95"]
        for i in range(16):
            blk += [f"v_cmp_gt_i32_e32 vcc, {8 * (i >> 2) + (i & 3)}, v95", f"v_cndmask_b32_e32 v{s + i}, v{s + i}, v116, vcc"]
        if LO:
            blk += [f"v_subrev_u32_e32 v96, %[maskfrom], %[lo{c}]", "v_add_u32_e32 v96, %[srem], v96",
                    f"v_subrev_u32_e32 v96, {32 * (kt + 1)}, v96"]
            for i in range(16):
                blk += [f"v_cmp_lt_i32_e32 vcc, {8 * (i >> 2) + (i & 3)}, v96", f"v_cndmask_b32_e32 v{s + i}, v{s + i}, v116, vcc"]
    blk.append(f"s_branch .Lpf_masked_{j}{kt}_%=")
    STUBS.append(blk)
    check = f"s_cmp_lt_i32 %[srem], {32 * (kt + 2)}\n\ts_cbranch_scc1 .Lpf_mask_{j}{kt}_%=\n"
    if LO:
        check += f"\ts_cmp_gt_i32 %[slo], {32 * (kt + 1)}\n\ts_cbranch_scc1 .Lpf_mask_{j}{kt}_%=\n"
    mx.append(Op(Ins(check + f".Lpf_masked_{j}{kt}_%=:", kind="salu", units=4 if LO else 2, n=4 if LO else 2,
                     reads=[f"v{S(nb, c) + i}" for c in range(NC) for i in range(16)]), MAX_GAP))
    for c in range(NC):
        s = S(nb, c)
        r = lambda i: f"v{s + i}"
        chain = [Ins(f"v_max3_f32 v{m[c]}, {r(0)}, {r(1)}, {r(2)}", reads=(r(0), r(1), r(2)), writes=(f"v{m[c]}",))]
        for i in range(3, 15, 2):
            chain.append(Ins(f"v_max3_f32 v{m[c]}, v{m[c]}, {r(i)}, {r(i + 1)}", reads=(f"v{m[c]}", r(i), r(i + 1)),
                             writes=(f"v{m[c]}",)))
        chain.append(Ins(f"v_max_f32_e32 v{m[c]}, v{m[c]}, {r(15)}", reads=(f"v{m[c]}", r(15)), writes=(f"v{m[c]}",)))
        for ins in chain:
            mx.append(Op(ins, MAX_GAP))
        mx.append(Op(Ins(f"v_mov_b32_e32 v{w[c]}, v{m[c]}", reads=(f"v{m[c]}",), writes=(f"v{w[c]}",)), MAX_GAP))
    for c in range(NC):
        mx.append(Op(Ins(f"v_permlane32_swap_b32_e32 v{m[c]}, v{w[c]}", kind="swap", reads=(f"v{m[c]}", f"v{w[c]}"),
                         writes=(f"v{m[c]}", f"v{w[c]}")), MAX_GAP))
        mx.append(Op(Ins(f"v_max_f32_e32 %[mx{c}], v{m[c]}, v{w[c]}", reads=(f"v{m[c]}", f"v{w[c]}")), MAX_GAP))
    # does a row's maximum exceed its reference by more than the slack?  (read at the start of the next subtile)
    # (with lower bounds a row may not have seen a key yet: its threshold thr is a large negative number until
    # it has, so that its first maximum, whatever its sign, becomes its reference)
    mx.append(Op(Ins(f"v_cmp_gt_f32_e64 s[60:61], %[mx0], {'%[thr0]' if LO else '%[slack]'}"), MAX_GAP))
    mx.append(Op(Ins(f"v_cmp_gt_f32_e64 s[62:63], %[mx1], {'%[thr1]' if LO else '%[slack]'}"), MAX_GAP))
    # (order: chain 0, copy 0, chain 1, copy 1, swap 0, max 0, swap 1, max 1: two instructions between a copy and its swap)
    streams["max"] = mx

    # ---- loads of tile j+3 into stage (j+3) % 4: table entries, then per 16-key group one K and one V load ----
    ldr = []
    dst_stage = (j + 3) % NSTAGE
    first = SYNC_GAP + 1 if kt == 0 else 0
    if kt == 0:
        # tile sT = t+3; past the last tile: tile 0 again (same loads and barriers for every wave, data unused)
        ldr.append(Op([Ins("s_cmp_lt_u32 %[sT], %[nreal]\n\ts_cselect_b32 s55, %[sT], 0", kind="salu", units=2, n=2),
                       Ins("s_lshl4_add_u32 s55, s55, %[tabA]", kind="salu"),
                       Ins("s_add_u32 %[sT], %[sT], 1", kind="salu"),
                       Ins("v_mov_b32_e32 v92, s55", writes=("v92",))], first))
        # (head_dim 128: a wave loads four rows of each of the tile's four 16-key groups; head_dim 64: eight rows of
        # two of them, groups w/2 and w/2 + 2 - the wave's first group is folded into tabA)
        read = "ds_read_b128 v[88:91], v92" if NG == 4 else "ds_read2_b32 v[88:89], v92 offset1:2"
        ldr.append(Op(Ins(read, kind="lds", reads=("v92",), issue="tab"), first))
        for n in range(NG):
            ldr.append(Op(Ins(f"v_readfirstlane_b32 s{40 + n}, v{88 + n}", reads=(f"v{88 + n}",), need=("tab",)), min(SYNC_GAP + 6, GAPS - 1)))
    groups = range(NG // 2) if kt == 0 else range(NG // 2, NG)
    for n in groups:
        e = min(SYNC_GAP + 8, GAPS - 1) if kt == 0 else 0
        # slot * row stride (64 bits), then per tensor: LDS destination into m0, pool base + offset, load.  The
        # two additions between the write of m0 and the load are the wait state that write needs.
        ldr.append(Op([Ins(f"s_mul_i32 s44, s{40 + n}, %[stride]", kind="salu"),
                       Ins(f"s_mul_hi_u32 s45, s{40 + n}, %[stride]", kind="salu")], e))
        dst = dst_stage * STAGE + n * 4096
        ld = "global_load_lds_dwordx4"
        ldr.append(Op(Ins(f"s_add_u32 m0, %[m0w], {dst}\n\ts_add_u32 s46, %[pklo], s44\n\ts_addc_u32 s47, %[pkhi], s45\n"
                          f"\t{ld} %[lanek], s[46:47]",
                          kind="vmem", units=5, n=4), e))
        ldr.append(Op(Ins(f"s_add_u32 m0, %[m0w], {dst + TENSOR}\n\ts_add_u32 s48, %[pvlo], s44\n\ts_addc_u32 s49, %[pvhi], s45\n"
                          f"\t{ld} %[lanev], s[48:49]",
                          kind="vmem", units=5, n=4), e))
    streams["ldr"] = ldr
    return mf, streams


def schedule(mf, streams, spare=0.6):
    """Places the other instructions into the 33 gaps around the products: earliest deadline first within the
    capacity of a gap, a stream's instructions in their order, everything due in a gap placed there."""
    total = sum(op.units for ops in streams.values() for op in ops)
    cap = total / (GAPS - 0.5) + spare
    order = ["chk", "lds", "pcs", "ldr", "max"]
    head = {k: 0 for k in streams}
    out = []
    for gap in range(GAPS):
        used = 0.0
        while True:
            ready = []
            for k in order:
                ops = streams.get(k, [])
                if head[k] < len(ops) and ops[head[k]].earliest <= gap:
                    ready.append((ops[head[k]].latest, order.index(k), k))
            if not ready:
                break
            ready.sort()
            limit = cap if gap < GAPS - 1 else 1e9
            placed = False
            for latest, _, k in ready:
                op = streams[k][head[k]]
                if latest > gap and used + op.units > limit + 1e-9:
                    continue
                out.extend(op.ins)
                used += op.units
                head[k] += 1
                placed = True
                break
            if not placed:
                break
        if gap < len(mf):
            out.append(mf[gap])
    for k, ops in streams.items():
        assert head[k] == len(ops), (k, head[k], len(ops))
    return out


def tile_body(ty, j):
    body = []
    for kt in range(2):
        mf, streams = subtile_ops(ty, j, kt)
        body += schedule(mf, streams)
    return body


def fixup():
    """Called before the barrier that publishes tile sP when that tile has rows that do not exist (past the
    context end, or in an absent block): table B holds, per 16-key group, the first such row (16 = none), and a
    lane clears its own 16 bytes of K and V when its row of the group is at or past it.  Every wave clears
    the rows it loaded itself, after the wait for its loads and before the barrier."""
    out = ["s_min_u32 s57, %[sP], %[captiles]",
           "s_lshl2_add_u32 s57, s57, %[tabB]",
           "v_mov_b32_e32 v99, s57",
           "ds_read_b32 v99, v99",
           "s_and_b32 s58, %[sP], 3",
           f"s_lshl_b32 s58, s58, {STAGE.bit_length() - 1}",
           "s_add_u32 s58, s58, %[m0w]",
           "s_waitcnt lgkmcnt(0)",
           "v_readfirstlane_b32 s57, v99",
           "v_add_u32_e32 v99, s58, %[lane16]"]
    if NG < 4:  # (the wave's first group is not group 0: its byte moves down to bit 0)
        out.append("s_lshr_b32 s57, s57, %[bshift]")
    for n in range(NG):
        out += [f"s_bfe_u32 s59, s57, {8 * (4 // NG) * n | (8 << 16)}",
                "v_cmp_le_u32_e32 vcc, s59, %[arow]",
                "s_nop 1",
                "s_and_saveexec_b64 s[52:53], vcc",
                f"ds_write_b128 v99, v[112:115] offset:{n * 4096}",
                f"ds_write_b128 v99, v[112:115] offset:{n * 4096 + TENSOR}",
                "s_mov_b64 exec, s[52:53]"]
    # The one 16-key group of a workgroup that reaches past the end of the pool (the last rows of the pool's last
    # block, when blocks are not multiples of 16 keys long): its direct loads fetched 16 rows from a slot where 16
    # exist, and the rows of it that exist are copied here, lane by lane, from where they are.  edgetile = its
    # tile (-1 = none), edgeslot = its first row, edgerows = how many exist, edgeofs = LDS offset of this wave's
    # load of that group (-1 = this wave loads no row of it).  (v88..v92 are free here: the table entries were
    # consumed in the previous tile, the next table address is formed behind the barrier.)
    out += ["s_cmp_lg_u32 %[sP], %[edgetile]",
            "s_cbranch_scc1 .Lpf_noedge_%=",
            "s_cmp_eq_u32 %[edgeofs], -1",
            "s_cbranch_scc1 .Lpf_noedge_%=",
            "s_mul_i32 s44, %[edgeslot], %[stride]",
            "s_mul_hi_u32 s45, %[edgeslot], %[stride]",
            "s_add_u32 s46, %[pklo], s44",
            "s_addc_u32 s47, %[pkhi], s45",
            "s_add_u32 s48, %[pvlo], s44",
            "s_addc_u32 s49, %[pvhi], s45",
            "v_cmp_gt_u32_e32 vcc, %[edgerows], %[arow]",
            "s_nop 1",
            "s_and_saveexec_b64 s[52:53], vcc",
            "global_load_dwordx4 v[88:91], %[lanek], s[46:47]",
            "v_add_u32_e32 v92, %[edgeofs], v99",
            "s_waitcnt vmcnt(0)",
            "ds_write_b128 v92, v[88:91]",
            "global_load_dwordx4 v[88:91], %[lanev], s[48:49]",
            "s_waitcnt vmcnt(0)",
            f"ds_write_b128 v92, v[88:91] offset:{TENSOR}",
            "s_mov_b64 exec, s[52:53]",
            ".Lpf_noedge_%=:"]
    out += ["s_waitcnt lgkmcnt(0)", "s_setpc_b64 s[50:51]"]
    return out


def add_waits(bodies):
    """Inserts s_waitcnt lgkmcnt(N) before consumers of LDS reads.  LDS reads return in order, so N = number of
    reads issued after the one needed.  The loop is simulated twice; the second round is the steady state (an
    entry from outside finds fewer reads outstanding than assumed, which only makes a wait return sooner)."""
    issued, pos, done = 0, {}, -1
    result = None
    for rnd in range(2):
        result = []
        for body in bodies:
            cur = []
            for ins in body:
                # (one wait per batch of reads: the first consumer of a batch waits for all of it, which has
                # long been issued by then, instead of one wait instruction per operand)
                fam = {g.rstrip("0123456789").rstrip("_") for g in ins.need}
                need = [q for g, q in pos.items() if g.rstrip("0123456789").rstrip("_") in fam]
                if need and max(need) > done:
                    n_after = issued - 1 - max(need)
                    n = min(15, n_after)
                    cur.append(Ins(f"s_waitcnt lgkmcnt({n})", kind="wait"))
                    done = issued - 1 - n
                if ins.kind == "lds":
                    if ins.issue:
                        pos[ins.issue] = issued
                    issued += 1
                cur.append(ins)
            result.append(cur)
    return result


def check_hazards(bodies):
    """Distances that the hardware does not interlock, checked over two rounds of the loop."""
    seq = [ins for _ in range(2) for body in bodies for ins in body]
    last_mfma_write, last_trans_write, last_valu_write = {}, {}, {}
    t = 0
    for ins in seq:
        if ins.kind != "mfma":
            for r in ins.reads + ins.writes:
                if r in last_mfma_write:
                    assert t - last_mfma_write[r] - 1 >= 19, (ins.text, r, t - last_mfma_write[r] - 1)
        if ins.kind in ("valu", "swap"):
            for r in ins.reads:
                if r in last_trans_write:
                    assert t - last_trans_write[r] - 1 >= 1, ("trans", ins.text)
        if ins.kind == "swap":
            for r in ins.reads:
                if r in last_valu_write:
                    assert t - last_valu_write[r] - 1 >= 2, ("swap", ins.text, t - last_valu_write[r] - 1)
        if ins.kind == "mfma":
            for r in ins.reads:  # operand words written by the vector unit
                if r in last_valu_write:
                    assert t - last_valu_write[r] - 1 >= 2, ("operand", ins.text)
        for r in ins.writes:
            last_mfma_write.pop(r, None)
            last_trans_write.pop(r, None)
            last_valu_write.pop(r, None)
            if ins.kind == "mfma":
                last_mfma_write[r] = t + ins.n - 1
            elif ins.kind == "trans":
                last_trans_write[r] = t + ins.n - 1
            else:
                last_valu_write[r] = t + ins.n - 1
        t += ins.n


def rescale(ty):
    """Called when the S^T values of a row (which are relative to the row's reference maximum) exceed the slack:
    the reference moves up by delta = max(maximum, 0) for both column tiles - the reference tiles, both S^T
    buffers (the current one was formed against the old reference; the other is dead and about to be
    overwritten) and the maximum itself shift by -delta, sums and accumulators (read from and written back to
    AGPRs) shrink by 2^-delta."""
    out = ["s_nop 7", "s_nop 7", "s_nop 7"]  # products still writing the accumulators
    for c in range(NC):
        if LO:
            # a row that had seen no key so far (thr still the large negative number; sum and accumulators zero)
            # takes its first maximum as reference whatever its sign, and nothing of it is scaled
            out += [f"v_max_f32_e32 v97, 0, %[mx{c}]",
                    f"v_cmp_lt_f32_e64 s[54:55], %[negbig], %[mx{c}]",       # this maximum is of visible keys
                    f"v_cndmask_b32_e64 v99, 0, %[mx{c}], s[54:55]",
                    f"v_cmp_eq_f32_e64 vcc, %[negbig], %[thr{c}]",            # no reference yet
                    "v_cndmask_b32_e32 v97, v97, v99, vcc",
                    "v_exp_f32_e64 v98, -v97",
                    f"v_sub_f32_e32 %[mx{c}], %[mx{c}], v97",
                    "v_mov_b32_e32 v99, %[slack]",
                    f"v_cndmask_b32_e64 %[thr{c}], %[thr{c}], v99, s[54:55]",
                    "v_cndmask_b32_e64 v98, v98, 1.0, vcc",
                    f"v_mul_f32_e32 %[l{c}], %[l{c}], v98"]
        else:
            out += [f"v_max_f32_e32 v97, 0, %[mx{c}]",
                    "v_exp_f32_e64 v98, -v97",
                    f"v_sub_f32_e32 %[mx{c}], %[mx{c}], v97",
                    "s_nop 0",
                    f"v_mul_f32_e32 %[l{c}], %[l{c}], v98"]
        for i in range(16):
            out.append(f"v_sub_f32_e32 v{CT(c) + i}, v{CT(c) + i}, v97")
        for buf in range(2):
            for i in range(16):
                out.append(f"v_sub_f32_e32 v{S(buf, c) + i}, v{S(buf, c) + i}, v97")
        for dt in range(DT):
            base = 16 * (DT * c + dt)
            for i in range(0, 16, 2):
                out += [f"v_accvgpr_read_b32 v93, a{base + i}", f"v_accvgpr_read_b32 v94, a{base + i + 1}",
                        "v_mul_f32_e32 v93, v93, v98", "v_mul_f32_e32 v94, v94, v98",
                        f"v_accvgpr_write_b32 a{base + i}, v93", f"v_accvgpr_write_b32 a{base + i + 1}, v94"]
    out += ["s_nop 7", "s_setpc_b64 s[50:51]"]
    return out


def loop_text(ty):
    del STUBS[:]
    bodies = [tile_body(ty, j) for j in range(NSTAGE)]
    bodies = add_waits(bodies)
    check_hazards(bodies)
    lines = []
    # prologue: addresses of stages 2 and 3 and the constants
    for ks in range(KS):
        lines.append(f"v_add_u32_e32 v{100 + ks}, {2 * STAGE}, %[kad{ks}]")
    for dt in range(DT):
        lines.append(f"v_add_u32_e32 v{108 + dt}, {2 * STAGE}, %[vad{dt}]")
    lines += [f"v_mov_b32_e32 v{r}, 0" for r in range(112, 116)]
    lines += ["v_mov_b32_e32 v116, 0xff800000",
              f"v_cmp_gt_f32_e64 s[60:61], %[mx0], {'%[thr0]' if LO else '%[slack]'}",
              f"v_cmp_gt_f32_e64 s[62:63], %[mx1], {'%[thr1]' if LO else '%[slack]'}", "s_waitcnt lgkmcnt(0)", "s_nop 3"]
    for j in range(NSTAGE):
        lines.append(f".Lpf_tile{j}_%=:")
        lines += [ins.text for ins in bodies[j]]
        # (ntiles counts the tiles after this one: the subtraction borrows behind the last)
        lines += ["s_sub_u32 %[srem], %[srem], 64"] + (["s_sub_u32 %[slo], %[slo], 64"] if LO else [])
        lines += ["s_sub_u32 %[ntiles], %[ntiles], 1", "s_cbranch_scc1 .Lpf_done_%="]
    lines.append("s_branch .Lpf_tile0_%=")
    for stub in STUBS:
        lines += stub
    lines.append(".Lpf_rescale_%=:")
    lines += rescale(ty)
    lines.append(".Lpf_fixup_%=:")
    lines += fixup()
    lines.append(".Lpf_done_%=:")
    lines.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    lines.append("s_nop 7")
    lines.append("s_nop 7")
    lines.append("s_nop 7")  # the last products have written the accumulators before anything reads them
    stats = {}
    for body in bodies:
        for ins in body:
            stats[ins.kind] = stats.get(ins.kind, 0) + ins.n
    return lines, stats


def c_string(lines):
    out = []
    for ln in lines:
        for part in ln.split("\n"):
            part = part.strip("\t")
            out.append('    "' + ("" if part.endswith(":") else "\\t") + part + '\\n"')
    return "\n".join(out)


def main():
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                               "prefill_mfma_loop.inc")
    parts = ["// Generated by gen_prefill_loop.py - do not edit.  The tile loops of prefill_asm_kernel (head_dim 128, 64, 32)",
             "// as inline assembly; the register map and the schedule are described in the generator.",
             ""]
    global LO
    for head_dim in (128, 64, 32):
        configure(head_dim)
        for lo in (False, True):
            LO = lo
            for name in ("bf16", "f16"):
                lines, stats = loop_text(Types(name))
                per_tile = {k: v // NSTAGE for k, v in sorted(stats.items())}
                what = f"{name}{', with lower bounds' if lo else ''}" + ("" if head_dim == 128 else f", head_dim {head_dim}")
                parts.append(f"// {what}: instructions per 64-key tile: {per_tile}")
                parts.append(f"#define PF_LOOP_ASM_{'' if head_dim == 128 else f'D{head_dim}_'}{name.upper()}{'_LO' if lo else ''} \\")
                body = c_string(lines).split("\n")
                parts.append(" \\\n".join(body))
                parts.append("")
    configure(128)
    with open(path, "w") as f:
        f.write("\n".join(parts))
    print("wrote", path)


if __name__ == "__main__":
    main()
