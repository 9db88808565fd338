#!/usr/bin/env python3
"""Writes prefill_d256_loop.inc: the subtile loop of the assembly instances of prefill_d256_kernel (head_dim 256,
block sizes that are multiples of 16) as one inline-assembly block per element type (bf16, fp16) and variant
(without / with lower bounds: sliding window, per-row first keys).

The instruction classes, the placement of the other instructions into the gaps around a subtile's 32 products,
the derivation of the `s_waitcnt lgkmcnt` values and the hazard checks are those of gen_prefill_loop.py; what
differs is the shape.  A wave owns one column tile of 32 query rows; a ring stage is one subtile of 32 keys and
holds V of tile s and K of tile s+1 (see prefill_d256.h); the loop is unrolled over the four ring slots.  Per
subtile g in slot j:
  products 0..15   S^T(g+1) = K(g+1) . Q^T, onto minus the reference maximum
  products 16..23  O^T += V^T(g, keys 0..15) . P^T     products 24..31: keys 16..31
  gaps 0..15       V^T reads of stage g (second k-step, and the second half of the first), the exponentials of S^T(g)
  gap 16           stage g+1 is published: this wave's loads of it have landed, rows that do not exist are cleared,
                   barrier; behind it the slot of stage g is free and takes the loads of stage g+4
  gaps 17..32      K reads of tile g+2 (stage g+1), the row maximum of S^T(g+1), the first V^T reads of stage g+1

Register map (per lane; the kernel pins its variables to the same registers):
  a[0:127]    O^T accumulators o[dt] at 16*dt
  a[128:191]  Q^T operands q[ks] at 128 + 4*ks
  a[192:255]  K operands ka[ks] at 192 + 4*ks
  v[0:31]     S^T: buffer b at 16*b; the subtile in slot j exponentiates buffer j & 1
  v[32:63]    V^T operands of the first k-step va0[dt] at 32 + 4*dt
  v[64:71]    P^T operand words
  v[80:87]    exponentials in flight, v[88:89] two table entries, v92 table address, v93 maximum, v95 its copy /
              a row's last visible key relative to the subtile, v[97:98] pair sums, v99 scratch
  v[100:111]  LDS read addresses of ring slots 2 and 3 (the operands hold those of slots 0 and 1)
  v[112:115]  zeros, v116 -inf
  v[118:133]  minus the rows' reference maximum (the accumulator input of the first S^T product)
  v[150:181]  V^T operands of the second k-step va1[dt] at 150 + 4*dt
  s[40:63]    scalars of the loads, the calls, the mask and the rescale check

Usage: python3 gen_prefill_loop_d256.py [output file]   (default: prefill_d256_loop.inc beside this script)
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from gen_prefill_loop import Ins, Op, Types, add_waits, areg, c_string, check_hazards, schedule, vreg  # noqa: E402

KS, DT = 16, 8
RB = 512                 # bytes of a K / V row
TENSOR = 32 * RB         # one tensor's 32 keys
STAGE = 2 * TENSOR       # K of tile s+1, then V of tile s
NSLOT = 4
SYNC_GAP = 16
LO = False                # the variant being generated also applies lower bounds (sliding window, per-row first keys)
CAP_TILES = 3072         # tiles the slot tables hold (kWdCapGroups / 2); the entries of four more groups follow, all absent
STUBS = []


def O(dt):
    return areg(16 * dt, 16)


def Q(ks):
    return areg(128 + 4 * ks, 4)


def KA(ks):
    return 192 + 4 * ks


def VA0(dt):
    return 32 + 4 * dt


def VA1(dt):
    return 150 + 4 * dt


S = lambda buf: 16 * buf
PP = 64
CT = 118


def k_addr(slot, ks):
    """(register, immediate) of the K operand read of k-step ks in a ring slot: k-steps 8..15 are 256 bytes behind 0..7."""
    reg = f"%[kad{ks & 7}]" if slot < 2 else f"v{100 + (ks & 7)}"
    return reg, (slot & 1) * STAGE + (ks >> 3) * 256


def v_addr(slot, dt):
    """The same for the V^T transpose read of d tile dt (tiles 4..7 are 256 bytes behind 0..3); the V part of a slot."""
    reg = f"%[vad{dt & 3}]" if slot < 2 else f"v{108 + (dt & 3)}"
    return reg, (slot & 1) * STAGE + (dt >> 2) * 256


def v_read(dst, slot, step, dt, group):
    """The two transposing reads of one V^T operand (keys 16*step .. +16 of the slot's tile, d tile dt)."""
    reg, imm = v_addr(slot, dt)
    base = imm + 16 * step * RB
    return [Ins(f"ds_read_b64_tr_b16 {vreg(dst, 2)}, {reg} offset:{base}", kind="lds"),
            Ins(f"ds_read_b64_tr_b16 {vreg(dst + 2, 2)}, {reg} offset:{base + 8 * RB}", kind="lds", issue=group)]


def subtile_ops(ty, j):
    cb, nb = j & 1, 1 - (j & 1)
    nslot = (j + 1) % NSLOT
    mf = []
    for ks in range(KS):
        s = S(nb)
        src_c = vreg(CT, 16) if ks == 0 else vreg(s, 16)
        mf.append(Ins(f"{ty.mfma} {vreg(s, 16)}, {areg(KA(ks), 4)}, {Q(ks)}, {src_c}", units=2, kind="mfma",
                      reads=[f"v{CT + i}" for i in range(16)] if ks == 0 else (),
                      writes=[f"v{s + i}" for i in range(16)], need=(f"ka{ks}",)))
    for step, va in ((0, VA0), (1, VA1)):
        for dt in range(DT):
            p = PP + 4 * step
            mf.append(Ins(f"{ty.mfma} {O(dt)}, {vreg(va(dt), 4)}, {vreg(p, 4)}, {O(dt)}", units=2, kind="mfma",
                          reads=[f"v{p + i}" for i in range(4)] + [f"v{va(dt) + i}" for i in range(4)],
                          need=(f"va{step}_{dt}",)))
    streams = {}

    # ---- rescale check ----
    chk = [Ins("s_mov_b64 vcc, s[60:61]", kind="salu"),
           Ins(f"s_cbranch_vccnz .Lwd_rescale_{j}_%=\n.Lwd_rescaled_{j}_%=:", kind="salu", n=1)]
    STUBS.append([f".Lwd_rescale_{j}_%=:", "s_call_b64 s[50:51], .Lwd_rescale_%=", f"s_branch .Lwd_rescaled_{j}_%="])
    streams["chk"] = [Op(chk, 0, 0)]

    # ---- LDS operand reads ----
    lds = []
    # stage g (slot j): the second half of the first k-step's V^T (consumed from product 20 on) and the second
    # k-step's (from product 24 on), all before the barrier that frees the slot
    for dt in range(4, DT):
        a, b = v_read(VA0(dt), j, 0, dt, f"va0_{dt}")
        lds += [Op(a, 2 * (dt - 4), 2 * (dt - 4)), Op(b, 2 * (dt - 4) + 1, 2 * (dt - 4) + 1)]
    for dt in range(DT):
        a, b = v_read(VA1(dt), j, 1, dt, f"va1_{dt}")
        lds += [Op(a, 2 * dt, 2 * dt), Op(b, 2 * dt + 1, 2 * dt + 1)]
    lds.sort(key=lambda op: op.earliest)
    # stage g+1 becomes visible: this wave's loads of it have landed (the 16 of stages g+2 and g+3 may be in
    # flight), its rows that do not exist are cleared, then every wave's
    lds.append(Op(Ins("s_waitcnt vmcnt(16)\n\ts_cmp_ge_u32 %[sP], %[splo]\n"
                      f"\ts_cbranch_scc1 .Lwd_fix_{j}_%=\n.Lwd_fixed_{j}_%=:\n"
                      "\ts_add_u32 %[sP], %[sP], 1\n\ts_barrier", kind="sync", units=5, n=5), SYNC_GAP, SYNC_GAP))
    STUBS.append([f".Lwd_fix_{j}_%=:", f"s_movk_i32 s58, {nslot * STAGE >> 8}", "s_call_b64 s[50:51], .Lwd_fixup_%=",
                  f"s_branch .Lwd_fixed_{j}_%="])
    # stage g+1 (slot j+1): K of tile g+2, one read per gap, and the first half of the first k-step's V^T
    for ks in range(KS):
        reg, imm = k_addr(nslot, ks)
        lds.append(Op(Ins(f"ds_read_b128 {areg(KA(ks), 4)}, {reg} offset:{imm}", kind="lds", issue=f"ka{ks}"),
                      17 + ks, 17 + ks))
        if ks >= 8:  # (the operand's last product of this subtile is number 16 + dt)
            dt, second = (ks - 8) >> 1, (ks - 8) & 1
            lds.append(Op(v_read(VA0(dt), nslot, 0, dt, f"va0_{dt}")[second], 17 + ks, 17 + ks))
    streams["lds"] = lds

    # ---- exponentials: piece n covers S^T values 2n, 2n+1 ----
    pcs = []

    def half_a(n):
        s0 = S(cb) + 2 * n
        ta, tb = 80 + 2 * (n % 4), 81 + 2 * (n % 4)
        return [Ins(f"v_exp_f32_e32 v{ta}, v{s0}", units=2, kind="trans", reads=(f"v{s0}",), writes=(f"v{ta}",)),
                Ins(f"v_exp_f32_e32 v{tb}, v{s0 + 1}", units=2, kind="trans", reads=(f"v{s0 + 1}",), writes=(f"v{tb}",))]

    def half_b(n):
        ta, tb = 80 + 2 * (n % 4), 81 + 2 * (n % 4)
        pr = 97 + (n & 1)
        out = [Ins(f"v_add_f32_e32 v{pr}, v{ta}, v{tb}", reads=(f"v{ta}", f"v{tb}"), writes=(f"v{pr}",))] + ty.pack(PP + n, ta, tb)
        if n >= 1:
            ppr = 97 + ((n - 1) & 1)
            out.append(Ins(f"v_add_f32_e32 %[l0], %[l0], v{ppr}", reads=(f"v{ppr}",)))
        if n == 7:
            out.append(Ins(f"v_add_f32_e32 %[l0], %[l0], v{pr}", reads=(f"v{pr}",)))
        return out

    def deadline(n):  # a whole gap before the product that reads the word
        return 14 if n < 4 else 22

    for n in range(8):
        pcs += [Op(ins, 0, deadline(n)) for ins in half_a(n)]
        if n >= 1:
            pcs += [Op(ins, 0, deadline(n - 1)) for ins in half_b(n - 1)]
    pcs += [Op(ins, 0, deadline(7)) for ins in half_b(7)]
    streams["pcs"] = pcs

    # ---- row maximum of S^T(g+1) (complete once product 15 has written it) ----
    # srem = maskfrom - 32*g: S^T(g+1) covers keys 32*(g+1) .. 32*(g+2)-1 and needs the mask if it reaches past
    # maskfrom: srem < 64.  Value i of a lane is key 8*(i/4) + i%4 of the subtile (+ 4*half, folded into lim).
    mx = []
    s = S(nb)
    blk = [f".Lwd_mask_{j}_%=:", "v_subrev_u32_e32 v95, %[maskfrom], %[lim0]", "v_add_u32_e32 v95, %[srem], v95",
           "v_subrev_u32_e32 v95, 32, v95"]
    for i in range(16):
        blk += [f"v_cmp_gt_i32_e32 vcc, {8 * (i >> 2) + (i & 3)}, v95", f"v_cndmask_b32_e32 v{s + i}, v{s + i}, v116, vcc"]
    if LO:
        # slo = (first key the wave's last row sees) - 32*g: S^T(g+1) also needs the mask if it starts below that
        # key: slo > 32; a value is then also masked below lo - first key of the subtile
        blk += ["v_subrev_u32_e32 v95, %[maskfrom], %[lo0]", "v_add_u32_e32 v95, %[srem], v95", "v_subrev_u32_e32 v95, 32, v95"]
        for i in range(16):
            blk += [f"v_cmp_lt_i32_e32 vcc, {8 * (i >> 2) + (i & 3)}, v95", f"v_cndmask_b32_e32 v{s + i}, v{s + i}, v116, vcc"]
    blk.append(f"s_branch .Lwd_masked_{j}_%=")
    STUBS.append(blk)
    check = f"s_cmp_lt_i32 %[srem], 64\n\ts_cbranch_scc1 .Lwd_mask_{j}_%=\n"
    if LO:
        check += f"\ts_cmp_gt_i32 %[slo], 32\n\ts_cbranch_scc1 .Lwd_mask_{j}_%=\n"
    mx.append(Op(Ins(check + f".Lwd_masked_{j}_%=:", kind="salu", units=4 if LO else 2, n=4 if LO else 2,
                     reads=[f"v{s + i}" for i in range(16)]), 21))
    r = lambda i: f"v{s + i}"
    chain = [Ins(f"v_max3_f32 v93, {r(0)}, {r(1)}, {r(2)}", reads=(r(0), r(1), r(2)), writes=("v93",))]
    for i in range(3, 15, 2):
        chain.append(Ins(f"v_max3_f32 v93, v93, {r(i)}, {r(i + 1)}", reads=("v93", r(i), r(i + 1)), writes=("v93",)))
    chain.append(Ins(f"v_max_f32_e32 v93, v93, {r(15)}", reads=("v93", r(15)), writes=("v93",)))
    for ins in chain:
        mx.append(Op(ins, 21))
    mx.append(Op(Ins("v_mov_b32_e32 v95, v93", reads=("v93",), writes=("v95",)), 21))
    mx.append(Op(Ins("s_nop 1", kind="salu", n=2), 21))  # (two wait states between the copy and the swap)
    mx.append(Op(Ins("v_permlane32_swap_b32_e32 v93, v95", kind="swap", reads=("v93", "v95"), writes=("v93", "v95")), 21))
    mx.append(Op(Ins("v_max_f32_e32 %[mx0], v93, v95", reads=("v93", "v95")), 21))
    # (with lower bounds a row may not have seen a key yet: its threshold thr is a large negative number until it
    # has, so that its first maximum, whatever its sign, becomes its reference)
    mx.append(Op(Ins(f"v_cmp_gt_f32_e64 s[60:61], %[mx0], {'%[thr0]' if LO else '%[slack]'}"), 21))
    streams["max"] = mx

    # ---- loads of stage g+4 into slot j: two table entries, then four K loads and four V loads ----
    # (table A holds two entries per tile; this wave's group is entry 2*tile + wave/2, folded into tabA.  The V
    # entry is tile sT's, the K entry tile sT+1's: two entries apart.  The tables run far enough past the last
    # tile for every tile the loop asks for.)
    ldr = []
    first = SYNC_GAP + 1
    ldr.append(Op([Ins(f"s_min_u32 s55, %[sT], {CAP_TILES}", kind="salu"),  # (tiles past the tables: entries of which nothing exists)
                   Ins("s_lshl3_add_u32 s55, s55, %[tabA]", kind="salu"),
                   Ins("s_add_u32 %[sT], %[sT], 1", kind="salu"),
                   Ins("v_mov_b32_e32 v92, s55", writes=("v92",))], first))
    ldr.append(Op(Ins("ds_read2_b32 v[88:89], v92 offset1:2", kind="lds", reads=("v92",), issue="tab"), first))
    for n in range(2):
        ldr.append(Op(Ins(f"v_readfirstlane_b32 s{40 + n}, v{88 + n}", reads=(f"v{88 + n}",), need=("tab",)), 22))
    dst = j * STAGE
    # (a direct load adds its immediate offset to the LDS and to the global address alike: with the global side
    # compensated in the per-lane offsets the four loads of a tensor share one write of m0; the additions between
    # that write and the first load are the wait states the write needs)
    for name, entry, lanes, ofs in (("k", 41, "lanek", 0), ("v", 40, "lanev", TENSOR)):
        ldr.append(Op([Ins(f"s_mul_i32 s44, s{entry}, %[stride]", kind="salu"),
                       Ins(f"s_mul_hi_u32 s45, s{entry}, %[stride]", kind="salu")], 24))
        ldr.append(Op(Ins(f"s_add_u32 m0, %[m0w], {dst + ofs}\n\ts_add_u32 s46, %[p{name}lo], s44\n\ts_addc_u32 s47, %[p{name}hi], s45\n"
                          + "\n".join(f"\tglobal_load_lds_dwordx4 %[{lanes}{n}], s[46:47] offset:{1024 * n}" for n in range(4)),
                          kind="vmem", units=7, n=7), 24))
    streams["ldr"] = ldr
    return mf, streams


def fixup():
    """Called before the barrier that publishes stage sP (K of tile sP+1, V of tile sP) when a tile from the first
    with rows that do not exist on is involved; s58 = the slot's byte offset / 256.  Table B holds, per 16-key
    group, the number of rows that exist; a lane clears its own 16 bytes of each of the four rows it loaded
    (rows arow, arow+2, arow+4, arow+6 of the group) that are at or past it."""
    out = [f"s_min_u32 s57, %[sP], {CAP_TILES}",
           "s_lshl1_add_u32 s57, s57, %[tabB]",   # V entry: group 2*sP + wave/2 (folded into tabB); K entry two on
           "v_mov_b32_e32 v99, s57",
           "ds_read_u8 v88, v99",
           "ds_read_u8 v89, v99 offset:2",
           "s_lshl_b32 s58, s58, 8",
           "s_add_u32 s58, s58, %[m0w]",
           "s_waitcnt lgkmcnt(0)",
           "v_readfirstlane_b32 s57, v88",    # rows of V of tile sP
           "v_readfirstlane_b32 s59, v89",    # rows of K of tile sP+1
           "v_add_u32_e32 v99, s58, %[lane16]"]
    # (v88, v89 and v92 are free here: the table entries were consumed in the previous subtile, the next table
    # address is formed behind the barrier; the pair sums v97 / v98 may be live)
    for n in range(4):
        out.append(f"v_add_u32_e32 v92, {2 * n}, %[arow]")
        for rows, ofs in (("s59", 0), ("s57", TENSOR)):
            out += [f"v_cmp_le_u32_e32 vcc, {rows}, v92",
                    "s_nop 1",
                    "s_and_saveexec_b64 s[52:53], vcc",
                    f"ds_write_b128 v99, v[112:115] offset:{n * 2 * RB + ofs}",
                    "s_mov_b64 exec, s[52:53]"]
    # The one 16-key group of a workgroup that reaches past the end of the pool (blocks that are not multiples of
    # 16 keys long: the last rows of the pool's last block): its direct loads fetched 16 rows from slot 0 instead,
    # and the rows of it that exist are copied here, lane by lane, from where they are - as K when the stage
    # holds its tile's K (tile sP+1), as V when it holds its V (tile sP).  edgetile = its tile for the waves that
    # load its rows (no tile for the others), edgeslot = its first row, edgerows = how many exist.
    # (v72..v75 are not used by the loop.)
    for name, tile_ofs, lanes, ofs in (("k", 1, "lanek", 0), ("v", 0, "lanev", TENSOR)):
        out += [f"s_add_u32 s56, %[sP], {tile_ofs}",
                "s_cmp_lg_u32 s56, %[edgetile]",
                f"s_cbranch_scc1 .Lwd_noedge_{name}_%=",
                "s_mul_i32 s44, %[edgeslot], %[stride]",
                "s_mul_hi_u32 s45, %[edgeslot], %[stride]",
                f"s_add_u32 s46, %[p{name}lo], s44",
                f"s_addc_u32 s47, %[p{name}hi], s45"]
        for n in range(4):
            out += [f"v_add_u32_e32 v92, {2 * n}, %[arow]",
                    "v_cmp_gt_u32_e32 vcc, %[edgerows], v92",
                    "s_nop 1",
                    "s_and_saveexec_b64 s[52:53], vcc",
                    f"global_load_dwordx4 v[72:75], %[{lanes}{n}], s[46:47] offset:{1024 * n}",
                    "s_waitcnt vmcnt(0)",
                    f"ds_write_b128 v99, v[72:75] offset:{n * 2 * RB + ofs}",
                    "s_mov_b64 exec, s[52:53]"]
        out.append(f".Lwd_noedge_{name}_%=:")
    out += ["s_waitcnt lgkmcnt(0)", "s_setpc_b64 s[50:51]"]
    return out


def rescale():
    """Called when the S^T values of a row (relative to its reference maximum) exceed the slack: the reference
    moves up by delta = max(maximum, 0): the reference tile, both S^T buffers and the maximum shift by -delta,
    the sum and the accumulators shrink by 2^-delta."""
    out = ["s_nop 7", "s_nop 7", "s_nop 7"]  # products still writing the accumulators
    if LO:
        # a row that had seen no key so far (thr still the large negative number; sum and accumulators zero)
        # takes its first maximum as reference whatever its sign, and nothing of it is scaled
        out += ["v_max_f32_e32 v97, 0, %[mx0]",
                "v_cmp_lt_f32_e64 s[54:55], %[negbig], %[mx0]",       # this maximum is of visible keys
                "v_cndmask_b32_e64 v99, 0, %[mx0], s[54:55]",
                "v_cmp_eq_f32_e64 vcc, %[negbig], %[thr0]",            # no reference yet
                "v_cndmask_b32_e32 v97, v97, v99, vcc",
                "v_exp_f32_e64 v98, -v97",
                "v_sub_f32_e32 %[mx0], %[mx0], v97",
                "v_mov_b32_e32 v99, %[slack]",
                "v_cndmask_b32_e64 %[thr0], %[thr0], v99, s[54:55]",
                "v_cndmask_b32_e64 v98, v98, 1.0, vcc",
                "v_mul_f32_e32 %[l0], %[l0], v98"]
    else:
        out += ["v_max_f32_e32 v97, 0, %[mx0]",
                "v_exp_f32_e64 v98, -v97",
                "v_sub_f32_e32 %[mx0], %[mx0], v97",
                "s_nop 0",
                "v_mul_f32_e32 %[l0], %[l0], v98"]
    for i in range(16):
        out.append(f"v_sub_f32_e32 v{CT + i}, v{CT + i}, v97")
    for buf in range(2):
        for i in range(16):
            out.append(f"v_sub_f32_e32 v{S(buf) + i}, v{S(buf) + i}, v97")
    for dt in range(DT):
        base = 16 * dt
        for i in range(0, 16, 2):
            out += [f"v_accvgpr_read_b32 v93, a{base + i}", f"v_accvgpr_read_b32 v95, a{base + i + 1}",
                    "v_mul_f32_e32 v93, v93, v98", "v_mul_f32_e32 v95, v95, v98",
                    f"v_accvgpr_write_b32 a{base + i}, v93", f"v_accvgpr_write_b32 a{base + i + 1}, v95"]
    out += ["s_nop 7", "s_setpc_b64 s[50:51]"]
    return out


def loop_text(ty):
    del STUBS[:]
    bodies = [schedule(*subtile_ops(ty, j)) for j in range(NSLOT)]
    bodies = add_waits(bodies)
    check_hazards(bodies)
    lines = []
    for ks in range(8):
        lines.append(f"v_add_u32_e32 v{100 + ks}, {2 * STAGE}, %[kad{ks}]")
    for dt in range(4):
        lines.append(f"v_add_u32_e32 v{108 + dt}, {2 * STAGE}, %[vad{dt}]")
    lines += [f"v_mov_b32_e32 v{r}, 0" for r in range(112, 116)]
    lines += ["v_mov_b32_e32 v116, 0xff800000", f"v_cmp_gt_f32_e64 s[60:61], %[mx0], {'%[thr0]' if LO else '%[slack]'}",
              "s_waitcnt lgkmcnt(0)", "s_nop 3"]
    for j in range(NSLOT):
        lines.append(f".Lwd_tile{j}_%=:")
        lines += [ins.text for ins in bodies[j]]
        lines += ["s_sub_u32 %[srem], %[srem], 32"] + (["s_sub_u32 %[slo], %[slo], 32"] if LO else [])
        lines += ["s_sub_u32 %[ntiles], %[ntiles], 1", "s_cbranch_scc1 .Lwd_done_%="]
    lines.append("s_branch .Lwd_tile0_%=")
    for stub in STUBS:
        lines += stub
    lines.append(".Lwd_rescale_%=:")
    lines += rescale()
    lines.append(".Lwd_fixup_%=:")
    lines += fixup()
    lines.append(".Lwd_done_%=:")
    lines += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_nop 7", "s_nop 7", "s_nop 7"]
    stats = {}
    for body in bodies:
        for ins in body:
            stats[ins.kind] = stats.get(ins.kind, 0) + ins.n
    return lines, stats


def operands():
    """The operand lists of the asm statement, pinned to the register map above."""
    outs = [f'"+{{a[{16 * dt}:{16 * dt + 15}]}}"(o[{dt}])' for dt in range(DT)]
    outs += ['"+{v[0:15]}"(sb0)', '"+{v[118:133]}"(ref)']
    outs += [f'"+{{a[{KA(ks)}:{KA(ks) + 3}]}}"(ka[{ks}])' for ks in range(KS)]
    # (Q^T is only read; as read-write operands the registers stay where they are when the statement sits in a loop)
    outs += [f'"+{{a[{128 + 4 * ks}:{131 + 4 * ks}]}}"(qreg[{ks}])' for ks in range(KS)]
    outs += [f'"+{{v[{VA0(dt)}:{VA0(dt) + 3}]}}"(va0[{dt}])' for dt in range(4)]
    outs += ['[mx0] "+&v"(mx)', '[l0] "+&v"(l_run)', '[ntiles] "+&s"(n_left)', '[sT] "+&s"(s_t)', '[sP] "+&s"(s_p)',
             '[srem] "+&s"(s_rem) MORE_OUT']
    ins = [f'[kad{ks}] "v"(kad[{ks}])' for ks in range(8)] + [f'[vad{dt}] "v"(vad[{dt}])' for dt in range(4)]
    ins += [f'[lanek{n}] "v"(lane_kb[{n}])' for n in range(4)] + [f'[lanev{n}] "v"(lane_vb[{n}])' for n in range(4)]
    ins += ['[lane16] "v"(lane16)', '[arow] "v"(arow_u)', '[lim0] "v"(lim)', '[slack] "s"(slack)', '[pklo] "s"(pklo)',
            '[pkhi] "s"(pkhi)', '[pvlo] "s"(pvlo)', '[pvhi] "s"(pvhi)', '[stride] "s"(stride)', '[m0w] "s"(m0w)',
            '[tabA] "s"(tab_a_w)', '[tabB] "s"(tab_b_w)', '[splo] "s"(sp_lo)', '[maskfrom] "s"(mask_from_u)',
            '[edgetile] "s"(edge_tile_u)', '[edgeslot] "s"(edge_slot_u)', '[edgerows] "s"(edge_rows_u) MORE_IN']
    clob = [f"v{r}" for r in list(range(16, 32)) + list(range(48, 118)) + list(range(150, 182))]
    clob += [f"s{r}" for r in range(40, 64)] + ["vcc", "scc", "memory"]

    def wrap(items, sep=", "):
        rows, cur = [], ""
        for it in items:
            if len(cur) + len(it) > 100:
                rows.append(cur)
                cur = ""
            cur += it + sep
        rows.append(cur[:-len(sep)])
        return " \\\n      ".join(rows)

    return (f"#define WD_LOOP_OPERANDS(MORE_OUT, MORE_IN) \\\n    : {wrap(outs)} \\\n    : {wrap(ins)} \\\n    : "
            + wrap([f'"{c}"' for c in clob]))


def main():
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                               "prefill_d256_loop.inc")
    parts = ["// Generated by gen_prefill_loop_d256.py - do not edit.  The subtile loop of prefill_d256_kernel's assembly",
             "// instances as inline assembly; the register map and the schedule are described in the generator.", ""]
    global LO
    for lo in (False, True):
        LO = lo
        for name in ("bf16", "f16"):
            lines, stats = loop_text(Types(name))
            per = {k: v // NSLOT for k, v in sorted(stats.items())}
            parts.append(f"// {name}{', with lower bounds' if lo else ''}: instructions per 32-key subtile: {per}")
            parts.append(f"#define WD_LOOP_ASM_{name.upper()}{'_LO' if lo else ''} \\")
            parts.append(" \\\n".join(c_string(lines).split("\n")))
            parts.append("")
    parts.append(operands())
    parts.append("")
    with open(path, "w") as f:
        f.write("\n".join(parts))
    print("wrote", path)


if __name__ == "__main__":
    main()
