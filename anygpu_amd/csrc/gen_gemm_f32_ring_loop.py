#!/usr/bin/env python3
"""Writes gemm_f32_ring_loop.inc and gemm_f32_ring_loop_64.inc: the main loops of the 128 x 128 and 64 x 64 fp32 GEMM
tile kernels of gemm_f32_ring.hpp (four waves, a 64 x 64 patch per wave as 2 x 2 tiles of v_mfma_f32_32x32x2_f32, or a
32 x 32 patch as one tile) as the text of one inline-assembly block, every instruction in issue order.

Why assembly: an fp32 MFMA takes 64 cycles, so the matrix cores are easy to keep busy on paper, but the kernel written
with builtins loses 7 - 14 % of their cycles around its barriers, one per 16-deep slab with every wave waiting for the
slowest.  Here the scheme of the fp16 four-wave kernels (gen_gemm_f16_ring_loop.py) is used: operands go from global
memory straight into LDS, three stages ahead, in whole 128-byte lines, and there is one barrier per 32-deep slab (4096
MFMA cycles), at mid-slab, when the loads of the slab after next have had two steps to land.

  a[0:63]                  accumulators, MFMA tile (i, j) of the wave's T x T patch in a[16 (T i + j) : + 15] (T = 2 or 1)
  v[128:143] / v[144:159]  A / B fragments of a 16-deep step (8 floats per tile row and lane), buffer 0; v[160:191] buffer 1
  v[96:99] / v[104:107]    byte offsets of this lane in the wave's four A / B loads of a slab (from a table in LDS)
  v[108:111] / v[112:115]  the lane's A / B fragment addresses inside a stage for step 0 (chunks c = 0, 1) and step 1
  v[116:119] / v[120:123]  the same in the stage being read: A step 0 (2), A step 1 (2) / B step 0 (2), B step 1 (2)
  s60 .. s62               LDS addresses of the stages of slabs t, t + 1, t + 2; s63 temporary of their rotation
  s65 slab counter, s66 last slab, s67 temporary, s[68:69] / s[70:71] global address of the A / B slab being requested,
  s72 / s73 where the wave's A / B loads of the current step go

A stage holds the 128 rows x 32 k (128-byte rows, 16-byte chunks swizzled by the row) of A and behind them of B for one
slab; stage s mod 3 holds slab s.  A lane (row r = lane % 32, half h = lane / 32) multiplies k = 16 h .. 16 h + 15 of a
slab, in two steps of 8; its chunks 4 h + 2 step + c sit at positions that differ from one another by an XOR of the low
address bits, so each of the four has its address register.  The mid-slab barrier of slab t frees the stage of slab t
(its last fragments were read during the first step), and the loads of slab t + 3 go there, half of them during the
second step of slab t and half during the first step of slab t + 1.

Operands of the block (named): vtab (VGPR: LDS address of the lane's table of load offsets, 256 bytes apart, A in rows
0 .. 3 and B in rows 8 .. 11), aaddr, baddr (VGPR: the lane's first fragment chunk of a slab inside a stage),
abaselo / abasehi, bbaselo / bbasehi (SGPR: global address of the wave's first row), lds0 (SGPR: LDS address of stage 0),
ldsa / ldsb (SGPR: offset of the wave's share of the A / B unit in a stage), slabs (SGPR: K / 32).

The 64 x 64 tile (T = 1) has units of 64 rows: two loads per wave, operand and slab, a stage of 16 KB, 8 MFMAs per step.

B stored [K, N] (the "kn" forms): a B unit is 32 k rows x 64 T n (rows of 256 T bytes, filled 2 or 4 rows per load); a
lane (column n = lane % 32 of its tile, half h) fetches its eight k of a step one float at a time down a column,
ds_read_b32 with the k row in the offset field.  Rows 16 apart (the two halves of the lanes) would fall on the same
banks, so the 16-byte chunks of rows 16 .. 31 are stored with bit 3 of their index flipped; for the tile column j that
bit is j, so each tile column has its address register (v112 + j inside a stage, v120 + j / v122 + j in the stages being
read).  A slab of B is 32 rows further on in memory (s64 and s74 hold the halves of that product); bsx (VGPR) is the
lane's flipped bit, bstep (SGPR) the bytes from one slab of B to the next.

Usage: gen_gemm_f32_ring_loop.py OUTPUT [64] [kn]
"""
import sys

S = ["s60", "s61", "s62"]
S_ROT, S_T, S_LAST, S_TMP, S_LDA, S_LDB = "s63", "s65", "s66", "s67", "s72", "s73"
A_CUR, B_CUR = "s[68:69]", "s[70:71]"
def frag_quad(base, c):
    return f"v[{base + 4 * c}:{base + 4 * c + 3}]"


def a_base(buf, i):
    return 128 + 32 * buf + 8 * i


def b_base(buf, j):
    return 144 + 32 * buf + 8 * j


def generate(T, kn=False):
    """T: MFMA tiles per wave and direction (2: tile 128 x 128, 1: tile 64 x 64); kn: B stored [K, N]"""
    lines = []
    ROWB = 256 * T                   # bytes of a [k][n] unit row
    STAGE = 2 * (64 * T) * 128       # bytes: A unit + B unit
    LOADS = 2 * T                    # per wave, operand and slab
    MFMAS = 8 * T * T                # per 16-deep step: 8 k pairs x T x T tiles

    def acc(i, j):
        r = 16 * (T * i + j)
        return f"a[{r}:{r + 15}]"

    def emit(s, comment=None):
        if isinstance(s, tuple):
            for x in s:
                emit(x)
            return
        lines.append((s, comment))

    # constants of the lane: fragment addresses inside a stage; v108 + 2 step + c for A, v112 + 2 step + c for B
    def a_const(step, c):
        return f"v{108 + 2 * step + c}"

    def b_const(step, c):
        return f"v{112 + c}" if kn else f"v{112 + 2 * step + c}"       # kn: c is the tile column

    def a_cur(step, c):
        return f"v{116 + 2 * step + c}"

    def b_cur(step, c):
        return f"v{120 + 2 * step + c}"

    def load_set(stage_reg, add):
        """where the loads of slab min(t + add, last) go and come from"""
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
        """half of the wave's eight loads of a slab as (M0 write, load) pairs: 0 the A loads, 1 the B loads"""
        out = []
        for q in range(LOADS):
            v = 96 + q + (8 if which == 1 else 0)
            out.append((f"s_add_u32 m0, {S_LDA if which == 0 else S_LDB}, {q * 1024}",
                        f"global_load_lds_dwordx4 v{v}, {A_CUR if which == 0 else B_CUR}"))
        return out

    def reads(buf, step):
        """the eight fragment reads of a step: tile row i of the patch lies 32 rows = 4096 bytes further on"""
        out = []
        for j in range(T):
            if kn:
                for e in range(8):
                    out.append(f"ds_read_b32 v{b_base(buf, j) + e}, {b_cur(step, j)} offset:{(8 * step + e) * ROWB}")
            else:
                for c in range(2):
                    out.append(f"ds_read_b128 {frag_quad(b_base(buf, j), c)}, {b_cur(step, c)} offset:{4096 * j}")
        for i in range(T):
            for c in range(2):
                out.append(f"ds_read_b128 {frag_quad(a_base(buf, i), c)}, {a_cur(step, c)} offset:{4096 * i}")
        return out

    def stage_addresses(step, stage_reg):
        return [f"v_add_u32 {a_cur(step, c)}, {stage_reg}, {a_const(step, c)}" for c in range(2)] + \
               [f"v_add_u32 {b_cur(step, c)}, {stage_reg}, {b_const(step, c)}" for c in range(T if kn else 2)]

    # ---- prologue: slabs 0 and 1 and the A loads of slab 2, fragments of the first step
    emit(f"s_mov_b32 {S_T}, 0", "prologue")
    emit(f"s_sub_u32 {S_LAST}, %[slabs], 1")
    for x in range(3):
        emit(f"s_add_u32 {S[x]}, %[lds0], {x * STAGE}")
    for q in range(LOADS):
        emit(f"ds_read_b32 v{96 + q}, %[vtab] offset:{256 * q}")
    for q in range(LOADS):
        emit(f"ds_read_b32 v{104 + q}, %[vtab] offset:{256 * (8 + q)}")
    emit("s_waitcnt lgkmcnt(0)")
    for step in range(2):
        for c in range(2):
            x = 16 * (2 * step + c)
            emit(f"v_xor_b32 {a_const(step, c)}, {x}, %[aaddr]" if x else f"v_mov_b32 {a_const(step, c)}, %[aaddr]")
            if not kn:
                emit(f"v_xor_b32 {b_const(step, c)}, {x}, %[baddr]" if x else f"v_mov_b32 {b_const(step, c)}, %[baddr]")
    if kn:
        for j in range(T):
            emit(f"v_xor_b32 {b_const(0, j)}, {128 * j}, %[bsx]")
            emit(f"v_add_u32 {b_const(0, j)}, %[baddr], {b_const(0, j)}")
    for slab in range(3):
        for ins in load_set(S[slab], slab):
            emit(ins)
        for m0w, ld in (loads(0) + loads(1)) if slab < 2 else loads(0):
            emit(m0w)
            emit("s_nop 0")
            emit(ld)
    for r in range(16 * T * T):
        emit(f"v_accvgpr_write_b32 a{r}, 0")
    emit(f"s_waitcnt vmcnt({3 * LOADS})", "slab 0 has landed")
    emit("s_barrier")
    # first half of slab 0 through the step-1 registers, then the step-0 registers point at its second half
    for ins in stage_addresses(0, S[0]):
        emit(ins)
    for ins in reads(0, 0):
        emit(ins)
    for ins in stage_addresses(1, S[0]):
        emit(ins)
    emit("s_waitcnt lgkmcnt(0)")

    # ---- main loop: one slab per trip.  Step 0 multiplies k step 0 of slab t (buffer 0) and reads k step 1 of slab t;
    # step 1 multiplies that (buffer 1) and reads k step 0 of slab t + 1.
    emit("1:", "main loop: one 32-deep slab per trip")
    for step in range(2):
        gaps = [[] for _ in range(MFMAS)]

        def place(entry, earliest):
            n = len(entry) if isinstance(entry, tuple) else 1
            # (an fp32 MFMA covers 64 cycles, sixteen issue slots)
            for cap in (1, 2, 3, 4, 6, 8, 10, 12):
                for g in range(earliest, MFMAS):
                    if sum(len(x) if isinstance(x, tuple) else 1 for x in gaps[g]) + n <= cap:
                        gaps[g].append(entry)
                        return g
            raise RuntimeError("the step has no room left")

        buf = step
        # the fragments of the next step: k step 1 of slab t in the stage of slab t, or k step 0 of slab t + 1
        step_reads = reads(buf ^ 1, 1 - step)
        spacing = 2 if T == 2 and not kn else 1
        for q, ins in enumerate(step_reads):
            gaps[spacing * q if spacing * (len(step_reads) - 1) < MFMAS else q * MFMAS // len(step_reads)].append(ins)
        # step 0: the B loads of slab t + 2; step 1: the A loads of slab t + 3
        last_load = 0
        every = 3 if T == 2 else 1
        for q, (m0w, ld) in enumerate(loads(1) if step == 0 else loads(0)):
            gaps[every * q + (1 if T == 2 else 0)].append(m0w)
            gaps[every * q + (2 if T == 2 else 1)].append(ld)
            last_load = every * q + (2 if T == 2 else 1)
        if step == 0:
            # once this step's loads are out: where the loads of slab t + 3 go (the stage of slab t) and come from; the
            # addresses of k step 0 in the stage of slab t + 1 (read during step 1)
            g = last_load + 1
            for ins in load_set(S[0], 3):
                g = place(ins, g)
            g = MFMAS // 2 + 1
            for ins in stage_addresses(0, S[1]):
                g = place(ins, g)
        else:
            # the stages move on by one slab, t advances; the addresses of k step 1 in the stage that now is slab t's
            g = 17 if T == 2 else 1
            for ins in [f"s_mov_b32 {S_ROT}, {S[0]}", f"s_mov_b32 {S[0]}, {S[1]}", f"s_mov_b32 {S[1]}, {S[2]}", f"s_mov_b32 {S[2]}, {S_ROT}",
                        f"s_add_u32 {S_T}, {S_T}, 1"] + stage_addresses(1, S[0]):
                g = place(ins, g + 1 if T == 2 else g)
        if step == 1:
            emit(f"s_waitcnt vmcnt({2 * LOADS})", "mid-slab: slab t + 1 has landed (the loads of slab t + 2 may be in flight)")
            emit("s_barrier")
        for m in range(MFMAS):
            e, t = m // (T * T), m % (T * T)
            i, j = t // T, t % T
            emit(f"v_mfma_f32_32x32x2_f32 {acc(i, j)}, v{b_base(buf, j) + e}, v{a_base(buf, i) + e}, {acc(i, j)}",
                 f"step {step}" if m == 0 else None)
            for ins in gaps[m]:
                emit(ins)
        emit("s_waitcnt lgkmcnt(0)")
    emit(f"s_cmp_lt_u32 {S_T}, %[slabs]")
    emit("s_cbranch_scc1 1b")
    emit("s_waitcnt vmcnt(0)", "nothing may still be writing LDS; the last MFMAs leave the pipeline before the accumulators are read")
    emit("s_barrier")
    for _ in range(5):
        emit("s_nop 15")
    return lines


if __name__ == "__main__":
    with open(sys.argv[1], "w") as f:
        f.write("// Written by gen_gemm_f32_ring_loop.py (the register plan and the schedule are explained there): do not edit.\n")
        for s, c in generate(1 if "64" in sys.argv[2:] else 2, "kn" in sys.argv[2:]):
            if c:
                f.write(f"// {c}\n")
            f.write(f'"{s}\\n\\t"\n')
