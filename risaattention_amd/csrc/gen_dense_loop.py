#!/usr/bin/env python3
"""Writes the hand-scheduled tile loops of the raw-score attention kernels for head dim 128 and
128-key tiles (every listed tile but the last) as gfx950 assembly: one `asm volatile` statement
each, whose operands are pinned to the registers chosen here.  Three programs: the dense launch,
the launch that walks a sparse pattern's tile lists, and the capturing launch of pattern
construction (the dense loop plus one statistics store per tile).

    python3 gen_dense_loop.py            # writes dense_, sparse_ and capture_loop_d128*.inc beside this file

Why assembly.  The loop owns the whole register file (256 vector registers at two wavefronts
per SIMD) and every phase reuses what the previous one has just left: the sixteen K fragments of
a tile are all requested at once into the registers of the P.V accumulators, the accumulator seeds
then land in the registers of the k-step that has just been multiplied, the seed block of the
score products borrows the V fragment registers, and the copies of the next tile are spread
between the matrix instructions.  The compiler's allocator does not find such a packing (it
serialises fragment reads behind `s_waitcnt lgkmcnt(0)` to save registers), and it cannot be told
where to put `s_setprio`.

Order of one tile (arithmetic identical to the C++ loop of attention_kernel.hpp, bit for bit):
  1. wait for the own copies, barrier; request 16 K fragments; fill the score seed block
  2. 16 score MFMAs, the next tile's 9 copies and the 16 accumulator-seed reads between them
  3. maxima of the seeded integers, tile maximum, online-softmax state (rescale when some row's
     maximum rises by more than 8)
  4. scaling pass: exponent arguments in place of the scores (two-cycle vector instructions; these
     leave no issue room beside a matrix instruction, so no matrix instruction sits here)
  5. exponentials and packs of key block 0; then the four value MFMAs of key block b between the
     exponentials, packs and row sums of block b+1 (four-cycle vector instructions co-issue with
     matrix instructions); the last four value MFMAs
  6. output update (two-cycle instructions), at the lowest wave priority: it is what the other
     wavefront of the SIMD overtakes.

The operands (see the asm statement in attention_kernel.hpp) and registers are listed below; the
program is checked on the CPU by tests/test_dense_loop_program.py, which interprets its scalar
side and compares every memory access with the C++ loop's.
"""
import argparse
import pathlib

STAGE = 2 * 16384 + 512 + 512  # bytes of one LDS stage: K tile, V tile, accumulator seeds, bias row
V_REGION = 16384               # V tile behind the K tile
SEED_REGION = 32768            # accumulator seeds behind both
SEED_BIAS = 2048               # the seed address register is 2 KiB ahead so that stage 1 stays within the 16-bit offset
COPIES = 4                     # 1 KiB copy instructions per wavefront and tile, for K and for V

# ---- vector registers ---------------------------------------------------------------------------
S = [0, 16, 32, 48]            # score accumulators, one block of 16 per 32-key block
ACC = [64, 80, 96, 112]        # P.V accumulators per 32-channel block; K fragments during the score product
O = [128, 144, 160, 176]       # outputs (operands, read and written)
Q = [192, 196, 200, 204]       # query fragments per k-step (operands)
VF = [208, 212, 216, 220]      # V fragments, one per channel block; score seed block during the score product
PK = [224, 228]                # packed probabilities of two key blocks in flight
T = [232, 233, 234, 235]       # exponentials in flight, temporaries of the output update
V_SC0, V_SC1, V_NEGM, V_MX0 = 236, 237, 238, 239
V_MX1, V_TMP, V_TMP2 = 228, 229, 230  # (the second probability block is free in that phase)
V_TSCALE, V_MRUN, V_DPART, V_ROWSUM, V_QSCALE, V_SEEDVAL = 240, 241, 242, 243, 244, 245
V_A = [246, 247, 248, 249]     # LDS address of this lane's fragment per k-step / key block (operands)
V_SEEDADDR = 250               # LDS address of this lane's accumulator seeds + SEED_BIAS (operand)
V_KC = [251, 252]              # lane share of the K copy source offsets, even / odd copies (operands)
V_VC = [253, 254]              # lane share of the V copy source offsets (operands)
# v255 is left to the compiler (it needs a vector register of its own for spilled scalar registers)

# ---- scalar registers (all clobbered) -------------------------------------------------------------
S_KPTR, S_VPTR, S_SUMPTR, S_KSPTR = 36, 38, 40, 42   # pairs: dense: sources of the next tile; sparse: bases of the head
S_COUNT, S_WAVE, S_LDS, S_QS2 = 44, 46, 47, 48
S_KS = 52                      # s[52:55]: the four K scales of the current tile
S_HALFMASK = 56                # pair: lanes 32..63
S_TMP, S_TMP2 = 58, 60         # pairs
S_KLDS, S_VLDS = 62, 63        # LDS offsets of this wave's copy slots in stage 0
S_VSTEP = 64                   # pair: bytes between the V rows of two copies (8 rows)
S_SAVEEXEC = 66                # pair
S_LIST = 68                    # pair: sparse: the query block's tile list
S_TNEXT, S_TAFTER, S_INDEX, S_LAST = 70, 71, 72, 73  # sparse: next tile, the one after it, its list index, last index
S_KWAVE, S_VWAVE = 74, 76      # pairs: sparse: this wave's share of the K and V sources
LAST_SGPR = 77
S_STATS, S_QLEN8, S_CAPEXEC = 78, 80, 82  # capture: pair: this wavefront's statistics rows of the tile; bytes per tile; pair: lanes that store
S_CAPNOW = 84                  # capture: pair: the lanes that store at the next statistics store (none before the first tile)
LAST_SGPR_CAPTURE = 85


class Emitter:
    """Instruction list with the bookkeeping the hardware leaves to the program: wait states after
    matrix and transcendental instructions, and the in-order counter of LDS reads."""

    def __init__(self):
        self.lines = []
        self.count = 0           # wait states issued so far (every instruction counts one)
        self.mfma_write = {}     # first register of a block -> count at the MFMA that wrote it last
        self.lds_queue = []      # destinations of outstanding ds_reads, oldest first
        self.trans_write = {}    # register -> count at the transcendental that wrote it
        self.valu_write = {}     # register -> count at its last vector write

    def raw(self, text):
        self.lines.append(text)

    def ins(self, text):
        self.lines.append(text)
        self.count += 1

    def comment(self, text):
        self.lines.append(f"; {text}")

    def nop(self, wait_states):
        while wait_states > 0:
            step = min(wait_states, 16)
            self.ins(f"s_nop {step - 1}")
            self.count += step - 1
            wait_states -= step

    def need_mfma_result(self, block, required=14):
        """A vector instruction is about to touch a block an 8-pass MFMA wrote (12 wait states on
        gfx950; 14 asked for)."""
        if block in self.mfma_write:
            distance = self.count - self.mfma_write[block]
            if distance < required:
                self.nop(required - distance)
            del self.mfma_write[block]

    def need_valu_result_for_mfma(self, registers, required=3):
        last = max((self.valu_write.get(r, -100) for r in registers), default=-100)
        if self.count - last < required:
            self.nop(required - (self.count - last))

    def need_trans(self, register):
        if register in self.trans_write:
            if self.count - self.trans_write[register] < 2:
                self.nop(1)
            del self.trans_write[register]

    def ds_read(self, dst, address, offset):
        assert 0 <= offset < 65536, offset
        self.ins(f"ds_read_b128 v[{dst}:{dst + 3}], v{address} offset:{offset}")
        self.lds_queue.append(dst)

    def wait_lds(self, dst):
        """Wait until the read into `dst` has landed (LDS reads return in order)."""
        if dst not in self.lds_queue:
            return
        index = self.lds_queue.index(dst)
        later = min(len(self.lds_queue) - 1 - index, 15)  # the counter holds 4 bits; waiting for more is safe
        self.ins(f"s_waitcnt lgkmcnt({later})")
        self.lds_queue = self.lds_queue[len(self.lds_queue) - later:] if later else []

    def mfma(self, dst, a, b, c):
        self.need_valu_result_for_mfma(list(range(a, a + 4)) + list(range(b, b + 4)))
        self.ins(f"v_mfma_i32_32x32x32_i8 v[{dst}:{dst + 15}], v[{a}:{a + 3}], v[{b}:{b + 3}], v[{c}:{c + 15}]")
        self.mfma_write[dst] = self.count

    def valu(self, text, writes=(), trans=False):
        self.ins(text)
        for register in writes:
            self.valu_write[register] = self.count
            if trans:
                self.trans_write[register] = self.count


def add64(e, pair, amount):
    e.ins(f"s_add_u32 s{pair}, s{pair}, {amount}")
    e.ins(f"s_addc_u32 s{pair + 1}, s{pair + 1}, 0")


def statistics_store(e):
    """Capturing launch: the statistics of the tile walked last — the row's sum of probability
    bytes (both halves of the wavefront) and the tile maximum, eight bytes per query, tile-major.
    Issued at the top of the next tile (and once behind the loop), where the row sum and the tile
    maximum are still in their registers: a store issued at the end of its own tile would be
    waited for at the next barrier, a few hundred cycles later, with the copies (stores and loads
    share the counter); issued here it has a whole tile to complete.  Before the first tile the
    lanes that store are none."""
    # (the row sum register is free by now: the swap may exchange halves in place; other
    # instructions stand where the lane swap needs wait states before and after it)
    e.valu(f"v_mov_b32_e32 v{T[1]}, v{V_ROWSUM}", [T[1]])
    e.valu(f"v_mbcnt_lo_u32_b32 v{T[0]}, -1, 0", [T[0]])
    e.valu(f"v_lshlrev_b32_e32 v{T[0]}, 3, v{T[0]}", [T[0]])  # lane * 8 (the lanes that store are 0..31)
    e.valu(f"v_permlane32_swap_b32_e32 v{V_ROWSUM}, v{T[1]}", [V_ROWSUM, T[1]])
    e.valu(f"v_mov_b32_e32 v{T[3]}, v{V_MX0}", [T[3]])
    e.nop(1)
    e.valu(f"v_add_u32_e32 v{T[2]}, v{V_ROWSUM}, v{T[1]}", [T[2]])
    e.ins(f"s_mov_b64 s[{S_SAVEEXEC}:{S_SAVEEXEC + 1}], exec")
    e.ins(f"s_mov_b64 exec, s[{S_CAPNOW}:{S_CAPNOW + 1}]")
    e.ins(f"global_store_dwordx2 v{T[0]}, v[{T[2]}:{T[3]}], s[{S_STATS}:{S_STATS + 1}]")
    e.ins(f"s_mov_b64 exec, s[{S_SAVEEXEC}:{S_SAVEEXEC + 1}]")
    e.ins(f"s_add_u32 s{S_STATS}, s{S_STATS}, s{S_QLEN8}")
    e.ins(f"s_addc_u32 s{S_STATS + 1}, s{S_STATS + 1}, 0")


def tile_body(e, stage, args, label):
    """One tile held in LDS stage `stage`; its copies fill the other stage with the next tile."""
    other = stage ^ 1
    base = stage * STAGE
    prio = args.prios
    e.comment(f"===== tile in stage {stage} =====")
    e.ins("s_waitcnt vmcnt(0) lgkmcnt(0)")  # own copies of this tile; K scales (and list entry) asked for a tile ago
    e.ins("s_barrier")
    e.ins(f"s_setprio {prio[0]}")
    for kk in range(4):
        for rb in range(4):
            e.ds_read(ACC[kk] + rb * 4, V_A[kk], base + rb * 4096)
    if args.capture:
        statistics_store(e)
    if args.sparse:
        # sources of the next listed tile: bases of the head (with this wave's share) + tile * stride
        e.ins(f"s_mov_b32 s{S_TNEXT}, s{S_TAFTER}")
        e.ins(f"s_lshl_b32 s{S_TMP}, s{S_TNEXT}, 14")
        e.ins(f"s_add_u32 s{S_TMP2}, s{S_KWAVE}, s{S_TMP}")
        e.ins(f"s_addc_u32 s{S_TMP2 + 1}, s{S_KWAVE + 1}, 0")
    # the score products start from the bits of 1.5 * 2^23 (one exact subtraction then turns an
    # accumulator into a float): the seed block borrows the V fragment registers, free in this phase
    for r in range(16):
        e.valu(f"v_mov_b32_e32 v{VF[0] + r}, v{V_SEEDVAL}", [VF[0] + r])

    copies = []  # the next tile's copies, interleaved with the matrix instructions

    def k_pointer():
        if not args.sparse:
            e.ins(f"s_mov_b64 s[{S_TMP2}:{S_TMP2 + 1}], s[{S_KPTR}:{S_KPTR + 1}]")

    def k_copy(i):
        def emit():
            e.ins(f"s_add_u32 m0, s{S_KLDS}, {other * STAGE + i * 1024}")
            e.ins("s_nop 0")
            # (no instruction offset: the hardware would add it to the LDS address as well)
            e.ins(f"global_load_lds_dwordx4 v{V_KC[i & 1]}, s[{S_TMP2}:{S_TMP2 + 1}]")
            if i < COPIES - 1:
                add64(e, S_TMP2, 1024)
        return emit

    def v_pointer():
        if args.sparse:
            e.ins(f"s_lshl_b32 s{S_TMP}, s{S_TNEXT}, 7")
            e.ins(f"s_add_u32 s{S_TMP}, s{S_VWAVE}, s{S_TMP}")
            e.ins(f"s_addc_u32 s{S_TMP + 1}, s{S_VWAVE + 1}, 0")
        else:
            e.ins(f"s_mov_b64 s[{S_TMP}:{S_TMP + 1}], s[{S_VPTR}:{S_VPTR + 1}]")

    def v_copy(i):
        def emit():
            e.ins(f"s_add_u32 m0, s{S_VLDS}, {other * STAGE + i * 1024}")
            e.ins("s_nop 0")
            e.ins(f"global_load_lds_dwordx4 v{V_VC[i & 1]}, s[{S_TMP}:{S_TMP + 1}]")
            if i < COPIES - 1:
                e.ins(f"s_add_u32 s{S_TMP}, s{S_TMP}, s{S_VSTEP}")
                e.ins(f"s_addc_u32 s{S_TMP + 1}, s{S_TMP + 1}, s{S_VSTEP + 1}")
        return emit

    def seed_copy():
        # wavefront 0, lanes 0..31: 512 bytes of accumulator seeds
        e.ins(f"s_cmp_lg_u32 s{S_WAVE}, 0")
        e.ins(f"s_cbranch_scc1 {label}_noseed")
        if args.sparse:
            e.ins(f"s_lshl_b32 s{S_TMP}, s{S_TNEXT}, 9")
            e.ins(f"s_add_u32 s{S_TMP}, s{S_SUMPTR}, s{S_TMP}")
            e.ins(f"s_addc_u32 s{S_TMP + 1}, s{S_SUMPTR + 1}, 0")
        e.ins(f"s_mov_b64 s[{S_SAVEEXEC}:{S_SAVEEXEC + 1}], exec")
        e.ins("s_mov_b64 exec, 0xffffffff")
        e.ins(f"s_add_u32 m0, s{S_LDS}, {other * STAGE + SEED_REGION}")
        e.ins("s_nop 0")
        e.ins(f"v_mbcnt_lo_u32_b32 v{T[0]}, -1, 0")
        e.ins(f"v_lshlrev_b32_e32 v{T[0]}, 4, v{T[0]}")  # lane * 16 (lanes 0..31)
        source = S_TMP if args.sparse else S_SUMPTR
        e.ins(f"global_load_lds_dwordx4 v{T[0]}, s[{source}:{source + 1}]")
        e.ins(f"s_mov_b64 exec, s[{S_SAVEEXEC}:{S_SAVEEXEC + 1}]")
        e.raw(f"{label}_noseed:")

    copies.append(k_pointer)
    copies += [k_copy(i) for i in range(COPIES)]
    copies.append(v_pointer)
    copies += [v_copy(i) for i in range(COPIES)]
    copies.append(seed_copy)
    for _ in range(min(args.lead_copies, len(copies))):
        copies.pop(0)()

    # ---- S^T = K Q^T -----------------------------------------------------------------------------
    for kk in range(4):
        for rb in range(4):
            e.wait_lds(ACC[kk] + rb * 4)
            e.mfma(S[rb], ACC[kk] + rb * 4, Q[kk], VF[0] if kk == 0 else S[rb])
            for _ in range(args.copies_per_mfma):
                if copies:
                    copies.pop(0)()
        # accumulator seeds of channel block kk into the registers this k-step has just left
        for b4 in range(4):
            e.ds_read(ACC[kk] + b4 * 4, V_SEEDADDR, base + SEED_REGION - SEED_BIAS + kk * 128 + b4 * 32)
    while copies:
        copies.pop(0)()
    if not args.sparse:
        add64(e, S_KPTR, 16384)
        add64(e, S_VPTR, 128)
        add64(e, S_SUMPTR, 512)

    # ---- K scales of this tile (scalar registers) -> score scales of this lane's two key groups ----
    e.ins(f"s_setprio {prio[1]}")
    e.valu(f"v_mov_b32_e32 v{V_TMP}, s{S_KS + 2}", [V_TMP])
    e.valu(f"v_mov_b32_e32 v{V_TMP2}, s{S_KS + 3}", [V_TMP2])
    e.valu(f"v_mov_b32_e32 v{V_SC0}, s{S_KS + 0}", [V_SC0])
    e.valu(f"v_mov_b32_e32 v{V_SC1}, s{S_KS + 1}", [V_SC1])
    e.valu(f"v_cndmask_b32_e64 v{V_SC0}, v{V_SC0}, v{V_TMP}, s[{S_HALFMASK}:{S_HALFMASK + 1}]", [V_SC0])
    e.valu(f"v_cndmask_b32_e64 v{V_SC1}, v{V_SC1}, v{V_TMP2}, s[{S_HALFMASK}:{S_HALFMASK + 1}]", [V_SC1])
    e.valu(f"v_mul_f32_e32 v{V_SC0}, v{V_QSCALE}, v{V_SC0}", [V_SC0])
    e.valu(f"v_mul_f32_e32 v{V_SC1}, v{V_QSCALE}, v{V_SC1}", [V_SC1])
    e.valu(f"v_mul_f32_e32 v{V_SC0}, s{S_QS2}, v{V_SC0}", [V_SC0])
    e.valu(f"v_mul_f32_e32 v{V_SC1}, s{S_QS2}, v{V_SC1}", [V_SC1])

    # ---- maxima of the seeded integer scores -------------------------------------------------------
    for rb in range(4):
        e.need_mfma_result(S[rb])
        evens = [S[rb] + i for i in range(16) if not i & 2]
        odds = [S[rb] + i for i in range(16) if i & 2]
        for target, registers in ((V_MX0, evens), (V_MX1, odds)):
            if rb == 0:
                e.valu(f"v_max_i32_e32 v{target}, v{registers[0]}, v{registers[1]}", [target])
                registers = registers[2:]
            while registers:
                e.valu(f"v_max3_i32 v{target}, v{target}, v{registers[0]}, v{registers[1]}", [target])
                registers = registers[2:]
    e.valu(f"v_sub_f32_e32 v{V_MX0}, v{V_MX0}, v{V_SEEDVAL}", [V_MX0])
    e.valu(f"v_sub_f32_e32 v{V_MX1}, v{V_MX1}, v{V_SEEDVAL}", [V_MX1])
    e.valu(f"v_mov_b32_e32 v{V_NEGM}, 0xc0ffd1be", [V_NEGM])  # -7.9943534f
    e.valu(f"v_fma_f32 v{V_MX0}, v{V_MX0}, v{V_SC0}, v{V_NEGM}", [V_MX0])
    e.valu(f"v_fma_f32 v{V_MX1}, v{V_MX1}, v{V_SC1}, v{V_NEGM}", [V_MX1])
    e.valu(f"v_max_f32_e32 v{V_MX0}, v{V_MX0}, v{V_MX1}", [V_MX0])
    e.valu(f"v_mov_b32_e32 v{V_MX1}, v{V_MX0}", [V_MX1])
    e.nop(2)
    e.valu(f"v_permlane32_swap_b32_e32 v{V_MX0}, v{V_MX1}", [V_MX0, V_MX1])  # the other half's maximum
    e.nop(2)
    e.valu(f"v_max_f32_e32 v{V_MX0}, v{V_MX0}, v{V_MX1}", [V_MX0])  # tile maximum - 7.99 of the row
    # ---- online-softmax state: the reference only moves when a tile maximum exceeds it by more than 8
    e.valu(f"v_add_f32_e32 v{V_TMP}, 0x41000000, v{V_MRUN}", [V_TMP])
    e.valu(f"v_cmp_gt_f32_e32 vcc, v{V_MX0}, v{V_TMP}")
    e.nop(4)
    e.ins(f"s_cbranch_vccz {label}_keep")
    e.valu(f"v_sub_f32_e32 v{V_TMP}, v{V_MRUN}, v{V_MX0}", [V_TMP])
    e.valu(f"v_exp_f32_e32 v{V_TMP}, v{V_TMP}", [V_TMP], trans=True)
    e.nop(1)
    e.valu(f"v_cndmask_b32_e32 v{V_TMP}, 1.0, v{V_TMP}, vcc", [V_TMP])
    e.valu(f"v_cndmask_b32_e32 v{V_MRUN}, v{V_MRUN}, v{V_MX0}, vcc", [V_MRUN])
    e.valu(f"v_mul_f32_e32 v{V_DPART}, v{V_DPART}, v{V_TMP}", [V_DPART])
    for cb in range(4):
        for i in range(16):
            e.valu(f"v_mul_f32_e32 v{O[cb] + i}, v{O[cb] + i}, v{V_TMP}", [O[cb] + i])
    e.raw(f"{label}_keep:")
    e.valu(f"v_sub_f32_e32 v{V_TSCALE}, v{V_MX0}, v{V_MRUN}", [V_TSCALE])
    e.valu(f"v_exp_f32_e32 v{V_TSCALE}, v{V_TSCALE}", [V_TSCALE], trans=True)
    e.valu(f"v_sub_f32_e32 v{V_NEGM}, 0, v{V_MX0}", [V_NEGM])

    # ---- V fragments of key block 0 (their latency hides behind the scaling pass) --------------------
    for cb in range(4):
        e.ds_read(VF[cb], V_A[0], base + V_REGION + cb * 4096)

    # ---- scaling pass: exponent arguments in place of the scores ---------------------------------------
    for rb in range(4):
        for i in range(16):
            e.valu(f"v_sub_f32_e32 v{S[rb] + i}, v{S[rb] + i}, v{V_SEEDVAL}", [S[rb] + i])
        for i in range(16):
            scale = V_SC1 if i & 2 else V_SC0
            e.valu(f"v_fma_f32 v{S[rb] + i}, v{S[rb] + i}, v{scale}, v{V_NEGM}", [S[rb] + i])
    e.valu(f"v_mov_b32_e32 v{V_ROWSUM}, 0", [V_ROWSUM])

    def pack_group(rb, b4, pk):
        """Four scores -> one register of signed probability bytes, and their sum."""
        registers = [S[rb] + b4 * 4 + r for r in range(4)]
        for r in range(4):
            e.valu(f"v_exp_f32_e32 v{T[r]}, v{registers[r]}", [T[r]], trans=True)
        for r in range(4):
            e.need_trans(T[r])
            previous = "0" if r == 0 else f"v{pk + b4}"
            e.valu(f"v_cvt_pk_u8_f32 v{pk + b4}, v{T[r]}, {r}, {previous}", [pk + b4])
        e.valu(f"v_sad_u8 v{V_ROWSUM}, v{pk + b4}, 0, v{V_ROWSUM}", [V_ROWSUM])
        e.valu(f"v_xor_b32_e32 v{pk + b4}, 0x80808080, v{pk + b4}", [pk + b4])

    e.ins(f"s_setprio {prio[2]}")
    for b4 in range(4):
        pack_group(0, b4, PK[0])
    for rb in range(1, 4):
        previous, current = PK[(rb - 1) & 1], PK[rb & 1]
        for cb in range(4):
            for b4 in range(4):
                e.wait_lds(ACC[cb] + b4 * 4)
            e.wait_lds(VF[cb])
            e.mfma(ACC[cb], VF[cb], previous, ACC[cb])
            e.ds_read(VF[cb], V_A[rb], base + V_REGION + cb * 4096)
            pack_group(rb, cb, current)
    for cb in range(4):
        e.wait_lds(VF[cb])
        e.mfma(ACC[cb], VF[cb], PK[1], ACC[cb])
    e.valu(f"v_cvt_f32_u32_e32 v{T[0]}, v{V_ROWSUM}", [T[0]])
    e.valu(f"v_fmac_f32_e32 v{V_DPART}, v{T[0]}, v{V_TSCALE}", [V_DPART])
    # ---- K scales (and list entry) of the next tile: waited for at the next barrier ------------------
    if args.sparse:
        e.ins(f"s_lshl_b32 s{S_TMP}, s{S_TNEXT}, 4")
        e.ins(f"s_add_u32 s{S_TMP}, s{S_KSPTR}, s{S_TMP}")
        e.ins(f"s_addc_u32 s{S_TMP + 1}, s{S_KSPTR + 1}, 0")
        e.ins(f"s_load_dwordx4 s[{S_KS}:{S_KS + 3}], s[{S_TMP}:{S_TMP + 1}], 0x0")
        e.ins(f"s_add_u32 s{S_INDEX}, s{S_INDEX}, 1")
        e.ins(f"s_min_u32 s{S_INDEX}, s{S_INDEX}, s{S_LAST}")
        e.ins(f"s_lshl_b32 s{S_TMP2}, s{S_INDEX}, 2")
        e.ins(f"s_add_u32 s{S_TMP2}, s{S_LIST}, s{S_TMP2}")
        e.ins(f"s_addc_u32 s{S_TMP2 + 1}, s{S_LIST + 1}, 0")
        e.ins(f"s_load_dword s{S_TAFTER}, s[{S_TMP2}:{S_TMP2 + 1}], 0x0")
    else:
        add64(e, S_KSPTR, 16)
        e.ins(f"s_load_dwordx4 s[{S_KS}:{S_KS + 3}], s[{S_KSPTR}:{S_KSPTR + 1}], 0x0")
    # ---- output update -------------------------------------------------------------------------------
    e.ins(f"s_setprio {prio[3]}")
    for cb in range(4):
        e.need_mfma_result(ACC[cb])
        for i in range(0, 16, 4):
            for j in range(4):
                e.valu(f"v_sub_f32_e32 v{T[j]}, v{ACC[cb] + i + j}, v{V_SEEDVAL}", [T[j]])
            for j in range(4):
                e.valu(f"v_fmac_f32_e32 v{O[cb] + i + j}, v{T[j]}, v{V_TSCALE}", [O[cb] + i + j])
    if args.capture:
        e.ins(f"s_mov_b64 s[{S_CAPNOW}:{S_CAPNOW + 1}], s[{S_CAPEXEC}:{S_CAPEXEC + 1}]")


def generate(args):
    e = Emitter()
    e.comment("set-up: operands into fixed scalar registers")
    e.ins(f"s_mov_b64 s[{S_KPTR}:{S_KPTR + 1}], %[kptr]")
    e.ins(f"s_mov_b64 s[{S_VPTR}:{S_VPTR + 1}], %[vptr]")
    e.ins(f"s_mov_b64 s[{S_SUMPTR}:{S_SUMPTR + 1}], %[sumptr]")
    e.ins(f"s_mov_b64 s[{S_KSPTR}:{S_KSPTR + 1}], %[ksptr]")
    e.ins(f"s_mov_b32 s{S_COUNT}, %[count]")
    e.ins(f"s_mov_b32 s{S_WAVE}, %[wave]")
    e.ins(f"s_mov_b32 s{S_QS2}, %[qs2]")
    e.ins(f"s_lshl_b32 s{S_VSTEP}, %[padded], 3")
    e.ins(f"s_mov_b32 s{S_VSTEP + 1}, 0")
    if args.sparse:
        e.ins(f"s_mov_b64 s[{S_LIST}:{S_LIST + 1}], %[list]")
    if args.capture:
        e.ins(f"s_mov_b64 s[{S_STATS}:{S_STATS + 1}], %[stats]")
        e.ins(f"s_mov_b32 s{S_QLEN8}, %[qlen8]")
        e.ins(f"s_mov_b64 s[{S_CAPEXEC}:{S_CAPEXEC + 1}], %[capexec]")
        # the store at the top of the first tile has no lanes and moves the pointer to tile 0
        e.ins(f"s_mov_b64 s[{S_CAPNOW}:{S_CAPNOW + 1}], 0")
        e.ins(f"s_sub_u32 s{S_STATS}, s{S_STATS}, s{S_QLEN8}")
        e.ins(f"s_subb_u32 s{S_STATS + 1}, s{S_STATS + 1}, 0")
    # LDS base: lane 0 of the seed address register holds base + SEED_BIAS
    e.ins(f"v_readfirstlane_b32 s{S_LDS}, v{V_SEEDADDR}")
    e.ins(f"s_sub_u32 s{S_LDS}, s{S_LDS}, {SEED_BIAS}")
    e.ins(f"s_mov_b32 s{S_HALFMASK}, 0")
    e.ins(f"s_mov_b32 s{S_HALFMASK + 1}, -1")
    # this wave's copy slots: wave * 4 KiB into the K tile / the V tile of a stage
    e.ins(f"s_lshl_b32 s{S_TMP}, s{S_WAVE}, 12")
    e.ins(f"s_add_u32 s{S_KLDS}, s{S_LDS}, s{S_TMP}")
    e.ins(f"s_add_u32 s{S_VLDS}, s{S_KLDS}, {V_REGION}")
    # this wave's sources: K advances wave * 4 KiB, V advances wave * 32 rows (4 copies of 8 rows)
    k_pair, v_pair = (S_KWAVE, S_VWAVE) if args.sparse else (S_KPTR, S_VPTR)
    e.ins(f"s_add_u32 s{k_pair}, s{S_KPTR}, s{S_TMP}")
    e.ins(f"s_addc_u32 s{k_pair + 1}, s{S_KPTR + 1}, 0")
    e.ins(f"s_lshl_b32 s{S_TMP2}, s{S_WAVE}, 2")
    e.ins(f"s_mul_hi_u32 s{S_TMP2 + 1}, s{S_TMP2}, s{S_VSTEP}")
    e.ins(f"s_mul_i32 s{S_TMP2}, s{S_TMP2}, s{S_VSTEP}")
    e.ins(f"s_add_u32 s{v_pair}, s{S_VPTR}, s{S_TMP2}")
    e.ins(f"s_addc_u32 s{v_pair + 1}, s{S_VPTR + 1}, s{S_TMP2 + 1}")
    if args.sparse:
        # list[0] is the tile whose copies are in flight, list[1] the first one this loop copies
        e.ins(f"s_load_dwordx2 s[{S_TMP}:{S_TMP + 1}], s[{S_LIST}:{S_LIST + 1}], 0x0")
        e.ins(f"s_mov_b32 s{S_LAST}, s{S_COUNT}")  # index of the last listed tile = number of tiles walked here
        e.ins(f"s_mov_b32 s{S_INDEX}, 1")
        e.ins("s_waitcnt lgkmcnt(0)")
        e.ins(f"s_mov_b32 s{S_TAFTER}, s{S_TMP + 1}")
        e.ins(f"s_lshl_b32 s{S_TMP}, s{S_TMP}, 4")
        e.ins(f"s_add_u32 s{S_TMP}, s{S_KSPTR}, s{S_TMP}")
        e.ins(f"s_addc_u32 s{S_TMP + 1}, s{S_KSPTR + 1}, 0")
        e.ins(f"s_load_dwordx4 s[{S_KS}:{S_KS + 3}], s[{S_TMP}:{S_TMP + 1}], 0x0")
    else:
        e.ins(f"s_load_dwordx4 s[{S_KS}:{S_KS + 3}], s[{S_KSPTR}:{S_KSPTR + 1}], 0x0")
    e.ins(f"v_mov_b32_e32 v{V_SEEDVAL}, 0x4b400000")
    e.raw("Lrisa_loop_%=:")
    tile_body(e, 0, args, "Lrisa_a_%=")
    e.ins(f"s_sub_u32 s{S_COUNT}, s{S_COUNT}, 1")
    e.ins(f"s_cmp_eq_u32 s{S_COUNT}, 0")
    e.ins("s_cbranch_scc1 Lrisa_done_%=")
    tile_body(e, 1, args, "Lrisa_b_%=")
    e.ins(f"s_sub_u32 s{S_COUNT}, s{S_COUNT}, 1")
    e.ins(f"s_cmp_lg_u32 s{S_COUNT}, 0")
    e.ins("s_cbranch_scc1 Lrisa_loop_%=")
    e.raw("Lrisa_done_%=:")
    e.ins("s_waitcnt lgkmcnt(0)")
    e.ins("s_setprio 0")
    if args.capture:
        statistics_store(e)  # of the last tile walked here
    return e


# (walks a tile list, stores the statistics of pattern construction, file stem)
PROGRAMS = ((False, False, "dense_loop_d128"), (True, False, "sparse_loop_d128"), (False, True, "capture_loop_d128"))


def render(args):
    """(program text, clobber list) as the two include files hold them."""
    e = generate(args)
    program = "".join('"{}\\n\\t"\n'.format(line.replace("\\", "\\\\").replace('"', '\\"')) for line in e.lines)
    operands = set(range(O[0], O[0] + 64)) | set(range(Q[0], Q[0] + 16)) | {V_MRUN, V_DPART, V_QSCALE}
    operands |= set(V_A) | {V_SEEDADDR} | set(V_KC) | set(V_VC)
    clobbered = [f"v{r}" for r in range(255) if r not in operands]
    clobbered += [f"s{r}" for r in range(36, (LAST_SGPR_CAPTURE if args.capture else LAST_SGPR) + 1)]
    clobbered += ["vcc", "scc", "m0", "memory"]
    return program, ", ".join(f'"{name}"' for name in clobbered) + "\n"


def parse(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--outdir", type=pathlib.Path, default=pathlib.Path(__file__).resolve().parent)
    parser.add_argument("--lead-copies", type=int, default=0, help="copy steps issued before the first matrix instruction")
    parser.add_argument("--copies-per-mfma", type=int, default=1, help="copy steps after every score matrix instruction")
    parser.add_argument("--prios", type=lambda text: [int(x) for x in text.split(",")], default=[0, 1, 2, 0],
                        help="wave priority in the score product, the maxima/scaling pass, the exponential rounds "
                             "and the output update (measured: 0,1,2,0 beats 0,2,1,2 by 2.5 %% and no priorities by 7 %%)")
    parser.set_defaults(sparse=False, capture=False)
    return parser.parse_args(argv)


def main():
    args = parse()
    for sparse, capture, stem in PROGRAMS:
        args.sparse, args.capture = sparse, capture
        program, clobbers = render(args)
        (args.outdir / f"{stem}.inc").write_text(program)
        (args.outdir / f"{stem}_clobbers.inc").write_text(clobbers)


if __name__ == "__main__":
    main()
