#!/usr/bin/env python3
"""Writes gemm_f16_ring_loop.inc and gemm_f16_ring_loop_kn.inc: the main loop of the 256 x 256 fp16 GEMM tile kernel of gemm_f16_ring.hpp (four waves, a
128 x 128 patch per wave) as the text of one inline-assembly block, every instruction in issue order.

Why assembly: with one wave per SIMD nothing hides a stall, and the 256 accumulator registers of a lane fill the AGPR file
exactly, which leaves the compiler's register allocator no room (it answered with copies between the two register files
or with spills).  Here every register is fixed:

  a[0:255]                 accumulators, MFMA tile (i, j) of the wave's 8 x 8 patch in a[4 (8 i + j) : + 3]
  v[128:159] / v[160:191]  B / A fragments of a 32-deep step, buffer 0;  v[192:223] / v[224:255]  buffer 1
  v[96:103]                byte offsets of this lane in the wave's eight A loads of a slab, v[104:111] the same for B
                           (computed by the kernel's C++ part, rows past the end of an operand clamped to its last row,
                           and handed over through a table in the fifth LDS unit, which the loop fills last)
  v112, v113               LDS addresses the fragment reads of the current step start from (A, B)
  v114, v115               fragment addresses of the second step of a slab (chunk + 4: address bit 6 flipped)
  s[60:64]                 LDS offsets of the units holding A(t), B(t), A(t+1), B(t+1) and of the free unit
  s65 slab counter, s66 last slab, s67 temporary, s[68:69] / s[70:71] global address of the A / B slab being requested,
  s72 unit that takes the B loads of the step

B stored [K, N] (the "kn" form): a B unit is 64 k rows x 256 n (512-byte rows, 16-byte chunks swizzled in pairs by the k
row), filled two rows per load, and a fragment is put together by two transposing reads (ds_read_b64_tr_b16, four k
each).  The swizzle permutes the eight column tiles of the patch differently in every lane, so each tile has an address
register of its own: v[80:87] inside a unit, v[88:95] in the unit being read; a slab of B is 64 rows further on in
memory, s73 holds the upper half of that product.

LDS holds five operand units of 32 KB: a unit is the 256 rows x 64 k (128-byte rows, 16-byte chunks swizzled by the row) of
A or of B for one 64-deep slab.  Operand slab n of the sequence A(0), B(0), A(1), B(1), ... lives in unit n mod 5.  While
slab t is multiplied, A(t), B(t), A(t+1), B(t+1) are resident and the fifth unit takes A(t+2) during the first 32-deep
step; at mid-slab, the one barrier of a slab, everybody has read A(t) and B(t), and B(t+2) goes where A(t) was during the
second step.  So a wave issues one direct load (1 KB: 8 rows x 128 bytes, whole cache lines) per eight MFMAs, all the
time, and every load has at least a step (64 MFMAs) to land.  Loads past the last slab fetch the last slab again into a
unit nobody reads, which keeps the loop free of branches and the counters uniform.

Under the 64 MFMAs of a step a wave issues the 16 fragment reads of the next step (one behind every second MFMA of the
first half), its 8 loads with their M0 writes, and the address arithmetic of the next step, never more than three
instructions behind one MFMA: with one wave per SIMD an MFMA covers 16 cycles, four instructions' worth of issue.

Operands of the block (named): vtab (VGPR: LDS address of the lane's table of 16 load offsets, 256 bytes apart), aaddr,
baddr (VGPR: LDS byte address of the lane's fragment chunk inside a unit, minus the wave's share), abaselo / abasehi,
bbaselo / bbasehi (SGPR: global address of the wave's first row), ldsw (SGPR: LDS address of the wave's 8 KB share of
unit 0), slabs (SGPR: K / 64); kn form also bsx (VGPR: the lane's swizzle, (k row bits) << 5) and bstep (SGPR: bytes
from one B slab to the next).

Smaller tiles ("8x4": 256 x 128, a 128 x 64 patch per wave; "4x4": 128 x 128, 64 x 64 patches) leave LDS room for three
whole stages of an A unit and a B unit, which is simpler: stage s mod 3 holds slab s, the mid-slab barrier of slab t frees
the stage of slab t (its last fragments were read during the first step), and the loads of slab t + 3 go there, half of
them during the second step of slab t and half during the first step of slab t + 1.  Registers as above except: s60 .. s62
LDS addresses of the stages of slabs t, t + 1, t + 2; s72 / s73 where the wave's A / B loads of the current step go;
v112 / v113 and v114 / v115 the fragment addresses of the first and of the second step, v116 / v117 the lane's fragment
addresses inside a stage with bit 6 flipped.  Operands: vtab, aaddr, baddr (inside a stage), abaselo .. bbasehi, slabs as
above, lds0 (SGPR: LDS address of stage 0), ldsa / ldsb (SGPR: offset of the wave's share of the A / B unit in a stage).

Usage: gen_gemm_f16_ring_loop.py OUTPUT [kn | 8x4 | 4x4 | 8x4kn | 4x4kn]
"""
import sys

UNIT = 32768
LOADS_AT = 5        # the load of a group of eight MFMAs goes behind this one, its M0 write behind the one before

O = ["s60", "s61", "s62", "s63", "s64"]
S_T, S_LAST, S_TMP, S_LD, S_HI = "s65", "s66", "s67", "s72", "s73"
A_CUR, B_CUR = "s[68:69]", "s[70:71]"
V_RA, V_RB, V_A1, V_B1 = "v112", "v113", "v114", "v115"
V_BUNIT, V_BCUR = 80, 88


def acc(i, j):
    r = 4 * (8 * i + j)
    return f"a[{r}:{r + 3}]"


def bfrag(buf, j, half=None):
    r = 128 + 64 * buf + 4 * j
    return f"v[{r}:{r + 3}]" if half is None else f"v[{r + 2 * half}:{r + 2 * half + 1}]"


def afrag(buf, i):
    r = 160 + 64 * buf + 4 * i
    return f"v[{r}:{r + 3}]"


def generate(kn):
    """the block's instructions as (text, comment) pairs; kn: B stored [K, N]"""
    lines = []
    # address arithmetic starts behind this MFMA (the reads of the step have been issued by then)
    extra_from = 47 if kn else 33

    def emit(s, comment=None):
        if isinstance(s, tuple):
            for x in s:
                emit(x)
            return
        lines.append((s, comment))

    def base_ops(cur, name, add):
        """global address of slab min(t + add, last) of one operand: 128 bytes per slab where k is contiguous, bstep
        bytes for B stored [K, N].  The add / add-with-carry pair is one entry: nothing that writes SCC may come
        between the two."""
        lo, hi = cur[2:-1].split(":")
        out = [f"s_add_u32 {S_TMP}, {S_T}, {add}", f"s_min_u32 {S_TMP}, {S_TMP}, {S_LAST}"]
        if kn and name == "bbase":
            out += [f"s_mul_hi_u32 {S_HI}, {S_TMP}, %[bstep]", f"s_mul_i32 {S_TMP}, {S_TMP}, %[bstep]",
                    (f"s_add_u32 s{lo}, %[{name}lo], {S_TMP}", f"s_addc_u32 s{hi}, %[{name}hi], {S_HI}")]
        else:
            out += [f"s_lshl_b32 {S_TMP}, {S_TMP}, 7",
                    (f"s_add_u32 s{lo}, %[{name}lo], {S_TMP}", f"s_addc_u32 s{hi}, %[{name}hi], 0")]
        return out

    def loads(operand, unit_reg):
        """the wave's eight loads of one operand slab as (M0 write, load) pairs"""
        out = []
        for q in range(8):
            v = 96 + q + (8 if operand == "b" else 0)
            out.append((f"s_add_u32 m0, {unit_reg}, {q * 1024}",
                        f"global_load_lds_dwordx4 v{v}, {A_CUR if operand == 'a' else B_CUR}"))
        return out

    def reads(buf, va, vb, second_half):
        """the fragment reads of a step.  k-contiguous operand: MFMA tile i of the patch lies 16 rows = 2048 bytes further
        on.  B stored [K, N]: per column tile its own address, the second 32-deep half of the slab 32 rows = 16 KB
        further on, the upper four k of a lane's eight 4 rows = 2 KB further on."""
        if kn:
            off = 16384 if second_half else 0
            out = [f"ds_read_b64_tr_b16 {bfrag(buf, q // 2, q % 2)}, v{V_BCUR + q // 2} offset:{off + 2048 * (q % 2)}" for q in range(16)]
        else:
            out = [f"ds_read_b128 {bfrag(buf, q)}, {vb} offset:{q * 2048}" for q in range(8)]
        out += [f"ds_read_b128 {afrag(buf, q)}, {va} offset:{q * 2048}" for q in range(8)]
        return out

    def b_unit_addresses(unit_reg):
        return [f"v_add_u32 v{V_BCUR + j}, {unit_reg}, v{V_BUNIT + j}" for j in range(8)]

    # ---- prologue: A(0), B(0), A(1), B(1) into units 0 .. 3, fragments of the first step
    emit(f"s_mov_b32 {S_T}, 0", "prologue")
    emit(f"s_sub_u32 {S_LAST}, %[slabs], 1")
    for x in range(5):
        emit(f"s_add_u32 {O[x]}, %[ldsw], {x * UNIT}")
    for q in range(16):
        emit(f"ds_read_b32 v{96 + q}, %[vtab] offset:{256 * q}")
    emit("s_waitcnt lgkmcnt(0)")
    emit(f"v_xor_b32 {V_A1}, 64, %[aaddr]")
    if kn:
        for j in range(8):
            emit(f"v_xor_b32 v{V_BUNIT + j}, {32 * j}, %[bsx]")
            emit(f"v_add_u32 v{V_BUNIT + j}, %[baddr], v{V_BUNIT + j}")
    else:
        emit(f"v_xor_b32 {V_B1}, 64, %[baddr]")
    for n, (operand, slab) in enumerate([("a", 0), ("b", 0), ("a", 1), ("b", 1)]):
        for ins in base_ops(A_CUR if operand == "a" else B_CUR, operand + "base", slab):
            emit(ins)
        for m0w, ld in loads(operand, O[n]):
            emit(m0w)
            emit("s_nop 0")
            emit(ld)
    for r in range(256):
        emit(f"v_accvgpr_write_b32 a{r}, 0")
    emit("s_waitcnt vmcnt(16)", "A(0), B(0) have landed")
    emit("s_barrier")
    emit(f"v_add_u32 {V_RA}, {O[0]}, %[aaddr]")
    if kn:
        for ins in b_unit_addresses(O[1]):
            emit(ins)
    else:
        emit(f"v_add_u32 {V_RB}, {O[1]}, %[baddr]")
    for ins in reads(0, V_RA, V_RB, False):
        emit(ins)
    emit(f"v_add_u32 {V_RA}, {O[0]}, {V_A1}", "addresses of the first step's reads (second half of slab 0), address of A(2)")
    if not kn:
        emit(f"v_add_u32 {V_RB}, {O[1]}, {V_B1}")
    for ins in base_ops(A_CUR, "abase", 2):
        emit(ins)
    emit("s_waitcnt lgkmcnt(0)")

    # ---- main loop: one slab per trip
    emit("1:", "main loop: one 64-deep slab per trip")
    for step in range(2):
        gaps = [[] for _ in range(64)]          # gaps[m]: what is issued behind MFMA m of the step
        buf = step
        # fragments of the next step: step 0 reads the second half of slab t, step 1 the first half of slab t + 1
        for q, ins in enumerate(reads(buf ^ 1, V_RA, V_RB, step == 0)):
            gaps[2 * q].append(ins)
        # step 0: A(t + 2) into the free unit; step 1: B(t + 2) into the unit A(t) has left
        if step == 1:
            gaps[0].append(f"s_mov_b32 {S_LD}, {O[0]}")
        for q, (m0w, ld) in enumerate(loads("a", O[4]) if step == 0 else loads("b", S_LD)):
            gaps[8 * q + LOADS_AT - 1].append(m0w)
            gaps[8 * q + LOADS_AT].append(ld)
        if step == 0:
            # read addresses of step 1 (first half of slab t + 1; in the kn form the B addresses stay for the first step
            # of the next trip, which reads the second half of the same unit); address of B(t + 2)
            extra = [f"v_add_u32 {V_RA}, {O[2]}, %[aaddr]"]
            extra += b_unit_addresses(O[3]) if kn else [f"v_add_u32 {V_RB}, {O[3]}, %[baddr]"]
            extra += base_ops(B_CUR, "bbase", 2)
        else:
            # the units move on by two operand slabs, t advances; read addresses of the next slab's first step; address of A(t + 3)
            extra = [f"s_mov_b32 {S_TMP}, {O[0]}", f"s_mov_b32 {O[0]}, {O[2]}", f"s_mov_b32 {O[2]}, {O[4]}", f"s_mov_b32 {O[4]}, {O[1]}",
                     f"s_mov_b32 {O[1]}, {O[3]}", f"s_mov_b32 {O[3]}, {S_TMP}", f"s_add_u32 {S_T}, {S_T}, 1",
                     f"v_add_u32 {V_RA}, {O[0]}, {V_A1}"]
            if not kn:
                extra.append(f"v_add_u32 {V_RB}, {O[1]}, {V_B1}")
            extra += base_ops(A_CUR, "abase", 2)
        for k, ins in enumerate(extra):
            gaps[extra_from + k].append(ins)
        if step == 1:
            emit("s_waitcnt vmcnt(8)", "mid-slab: A(t+1), B(t+1) have landed (the loads of A(t+2) may be in flight)")
            emit("s_barrier")
        for m in range(64):
            # row by row through the patch, every other row backwards, so that one operand stays when the row changes
            i, j = m // 8, m % 8
            if i % 2 == 1:
                j = 7 - j
            emit(f"v_mfma_f32_16x16x32_f16 {acc(i, j)}, {bfrag(buf, j)}, {afrag(buf, i)}, {acc(i, j)}",
                 f"step {step}" if m == 0 else None)
            for ins in gaps[m]:
                emit(ins)
        emit("s_waitcnt lgkmcnt(0)")
    emit(f"s_cmp_lt_u32 {S_T}, %[slabs]")
    emit("s_cbranch_scc1 1b")
    emit("s_waitcnt vmcnt(0)", "nothing may still be writing LDS; the last MFMAs leave the pipeline before the accumulators are read")
    emit("s_barrier")
    emit("s_nop 15")
    emit("s_nop 15")
    return lines


def generate_three_stages(tm, tn, kn=False):
    """the block for a patch of tm x tn MFMA tiles per wave (tile 32 tm x 32 tn), three LDS stages; kn: B stored [K, N]
    (a B unit of 64 k rows x 32 tn n, fragments by transposing reads through one address register per column tile, as in
    the kn form of the 256 x 256 tile; s64 and s74 hold the halves of the slab's byte offset)"""
    lines = []
    bm, bn = 32 * tm, 32 * tn
    stage = (bm + bn) * 128
    la, lb = bm // 32, bn // 32                 # loads per wave and slab
    half = (la + lb) // 2
    load_list = [("a", q) for q in range(la)] + [("b", q) for q in range(lb)]
    S = ["s60", "s61", "s62"]
    S_ROT, S_LDA, S_LDB = "s63", "s72", "s73"
    V_RA0, V_RB0, V_RA1, V_RB1, V_A64, V_B64 = "v112", "v113", "v114", "v115", "v116", "v117"
    mfmas = tm * tn

    def emit(s, comment=None):
        if isinstance(s, tuple):
            for x in s:
                emit(x)
            return
        lines.append((s, comment))

    def tile_acc(i, j):
        r = 4 * (tn * i + j)
        return f"a[{r}:{r + 3}]"

    def load_set(stage_reg, add):
        """where the loads of slab min(t + add, last) go and come from: entries of one or two instructions"""
        out = [f"s_add_u32 {S_LDA}, {stage_reg}, %[ldsa]", f"s_add_u32 {S_LDB}, {stage_reg}, %[ldsb]",
               f"s_add_u32 {S_TMP}, {S_T}, {add}", f"s_min_u32 {S_TMP}, {S_TMP}, {S_LAST}"]
        if kn:
            out += ["s_mul_hi_u32 s64, " + S_TMP + ", %[bstep]", "s_mul_i32 s74, " + S_TMP + ", %[bstep]",
                    ("s_add_u32 s70, %[bbaselo], s74", "s_addc_u32 s71, %[bbasehi], s64")]
        out += [f"s_lshl_b32 {S_TMP}, {S_TMP}, 7", ("s_add_u32 s68, %[abaselo], " + S_TMP, "s_addc_u32 s69, %[abasehi], 0")]
        if not kn:
            out.append(("s_add_u32 s70, %[bbaselo], " + S_TMP, "s_addc_u32 s71, %[bbasehi], 0"))
        return out

    def loads(which):
        out = []
        for operand, q in load_list[:half] if which == 0 else load_list[half:]:
            v = 96 + q + (8 if operand == "b" else 0)
            out.append((f"s_add_u32 m0, {S_LDA if operand == 'a' else S_LDB}, {q * 1024}",
                        f"global_load_lds_dwordx4 v{v}, {A_CUR if operand == 'a' else B_CUR}"))
        return out

    row_kn = 64 * tn                            # bytes of a [k][n] unit row

    def reads(buf, va, vb, second_half=False):
        if kn:
            off = 32 * row_kn if second_half else 0
            out = [f"ds_read_b64_tr_b16 {bfrag(buf, q // 2, q % 2)}, v{V_BCUR + q // 2} offset:{off + 4 * row_kn * (q % 2)}" for q in range(2 * tn)]
        else:
            out = [f"ds_read_b128 {bfrag(buf, q)}, {vb} offset:{q * 2048}" for q in range(tn)]
        out += [f"ds_read_b128 {afrag(buf, q)}, {va} offset:{q * 2048}" for q in range(tm)]
        return out

    def b_stage_addresses(stage_reg):
        return [f"v_add_u32 v{V_BCUR + j}, {stage_reg}, v{V_BUNIT + j}" for j in range(tn)]

    # ---- prologue: slabs 0 and 1 and the first half of the loads of slab 2, fragments of the first step
    emit(f"s_mov_b32 {S_T}, 0", "prologue")
    emit(f"s_sub_u32 {S_LAST}, %[slabs], 1")
    for x in range(3):
        emit(f"s_add_u32 {S[x]}, %[lds0], {x * stage}")
    for q in range(la):
        emit(f"ds_read_b32 v{96 + q}, %[vtab] offset:{256 * q}")
    for q in range(lb):
        emit(f"ds_read_b32 v{104 + q}, %[vtab] offset:{256 * (8 + q)}")
    emit("s_waitcnt lgkmcnt(0)")
    emit(f"v_xor_b32 {V_A64}, 64, %[aaddr]")
    if kn:
        for j in range(tn):
            emit(f"v_xor_b32 v{V_BUNIT + j}, {32 * j}, %[bsx]")
            emit(f"v_add_u32 v{V_BUNIT + j}, %[baddr], v{V_BUNIT + j}")
    else:
        emit(f"v_xor_b32 {V_B64}, 64, %[baddr]")
    for slab in range(3):
        for ins in load_set(S[slab], slab):
            emit(ins)
        for m0w, ld in (loads(0) + loads(1)) if slab < 2 else loads(0):
            emit(m0w)
            emit("s_nop 0")
            emit(ld)
    for r in range(4 * mfmas):
        emit(f"v_accvgpr_write_b32 a{r}, 0")
    emit(f"s_waitcnt vmcnt({la + lb + half})", "slab 0 has landed")
    emit("s_barrier")
    emit(f"v_add_u32 {V_RA1}, {S[0]}, %[aaddr]")
    if kn:
        for ins in b_stage_addresses(S[0]):
            emit(ins)
    else:
        emit(f"v_add_u32 {V_RB1}, {S[0]}, %[baddr]")
    for ins in reads(0, V_RA1, V_RB1):
        emit(ins)
    emit(f"v_add_u32 {V_RA0}, {S[0]}, {V_A64}")
    if not kn:
        emit(f"v_add_u32 {V_RB0}, {S[0]}, {V_B64}")
    emit("s_waitcnt lgkmcnt(0)")

    # ---- main loop: one slab per trip
    emit("1:", "main loop: one 64-deep slab per trip")
    for step in range(2):
        gaps = [[] for _ in range(mfmas)]

        def place(entry, earliest):
            """behind the first MFMA from `earliest` on that has fewer than two instructions behind it (three, four if none has)"""
            n = len(entry) if isinstance(entry, tuple) else 1
            for cap in (2, 3, 4):
                for g in range(earliest, mfmas):
                    if sum(len(x) if isinstance(x, tuple) else 1 for x in gaps[g]) + n <= cap:
                        gaps[g].append(entry)
                        return g
            raise RuntimeError("the step has no room left")

        buf = step
        # fragments of the next step: step 0 reads the second half of slab t, step 1 the first half of slab t + 1
        step_reads = reads(buf ^ 1, V_RA0 if step == 0 else V_RA1, V_RB0 if step == 0 else V_RB1, step == 0)
        spacing = 2 if 2 * (len(step_reads) - 1) < mfmas else 1
        for q, ins in enumerate(step_reads):
            gaps[spacing * q].append(ins)
        # step 0: the second half of the loads of slab t + 2; step 1: the first half of the loads of slab t + 3
        every = max(2, (mfmas - 10) // half)
        last_load = 0
        for q, (m0w, ld) in enumerate(loads(1) if step == 0 else loads(0)):
            gaps[every * q].append(m0w)
            gaps[every * q + 1].append(ld)
            last_load = every * q + 1
        if step == 0:
            # fragment addresses of step 1; once this step's loads are out, where the loads of slab t + 3 go (the stage of
            # slab t) and come from
            g = place(f"v_add_u32 {V_RA1}, {S[1]}, %[aaddr]", 1)
            if not kn:
                g = place(f"v_add_u32 {V_RB1}, {S[1]}, %[baddr]", g)
            g = last_load + 1
            for ins in load_set(S[0], 3):
                g = place(ins, g)
            if kn:
                # (the B addresses serve this step's reads first; the new ones stay for the first step of the next trip,
                # which reads the second half of the same stage)
                g = spacing * (2 * tn - 1) + 1
                for ins in b_stage_addresses(S[1]):
                    g = place(ins, g)
        else:
            # the stages move on by one slab, t advances; fragment addresses of the next trip's first step
            g = 1
            for ins in [f"s_mov_b32 {S_ROT}, {S[0]}", f"s_mov_b32 {S[0]}, {S[1]}", f"s_mov_b32 {S[1]}, {S[2]}", f"s_mov_b32 {S[2]}, {S_ROT}",
                        f"s_add_u32 {S_T}, {S_T}, 1", f"v_add_u32 {V_RA0}, {S[0]}, {V_A64}"] + ([] if kn else [f"v_add_u32 {V_RB0}, {S[0]}, {V_B64}"]):
                g = place(ins, g + 1)
        if step == 1:
            emit(f"s_waitcnt vmcnt({la + lb})", "mid-slab: slab t + 1 has landed (the loads of slab t + 2 may be in flight)")
            emit("s_barrier")
        for m in range(mfmas):
            i, j = m // tn, m % tn
            if i % 2 == 1:
                j = tn - 1 - j
            emit(f"v_mfma_f32_16x16x32_f16 {tile_acc(i, j)}, {bfrag(buf, j)}, {afrag(buf, i)}, {tile_acc(i, j)}",
                 f"step {step}" if m == 0 else None)
            for ins in gaps[m]:
                emit(ins)
        emit("s_waitcnt lgkmcnt(0)")
    emit(f"s_cmp_lt_u32 {S_T}, %[slabs]")
    emit("s_cbranch_scc1 1b")
    emit("s_waitcnt vmcnt(0)", "nothing may still be writing LDS; the last MFMAs leave the pipeline before the accumulators are read")
    emit("s_barrier")
    emit("s_nop 15")
    emit("s_nop 15")
    return lines


if __name__ == "__main__":
    form = sys.argv[2] if len(sys.argv) > 2 else ""
    with open(sys.argv[1], "w") as f:
        f.write("// Written by gen_gemm_f16_ring_loop.py (the register plan and the schedule are explained there): do not edit.\n")
        kn = form.endswith("kn")
        patch = form[:-2] if kn else form
        for s, c in (generate_three_stages(*(int(x) for x in patch.split("x")), kn) if "x" in patch else generate(kn)):
            if c:
                f.write(f"// {c}\n")
            f.write(f'"{s}\\n\\t"\n')
