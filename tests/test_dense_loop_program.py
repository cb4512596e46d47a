"""The hand-scheduled tile loops (risaattention_amd/csrc/dense_loop_d128.inc, sparse_loop_d128.inc)
checked on the CPU: the committed text is what the generator writes, and an interpreter of the
program's scalar side (pointer arithmetic, M0, EXEC, the loop counter, the tile list) compares
every memory access of a model launch with what the C++ tile loop of attention_kernel.hpp does
for the same wavefront: source and LDS destination of every lane of every global->LDS copy, the
address of every LDS fragment read and the register block it lands in, the scalar loads of K
scales and list entries, the trip count and the number of barriers.  What the GPU tests then add
is the arithmetic (bit-identical outputs with the loop the compiler schedules)."""

import importlib.util
import random
import re
from pathlib import Path

import pytest

CSRC = Path(__file__).resolve().parents[1] / "risaattention_amd" / "csrc"
STAGE = 2 * 16384 + 512 + 512
D = CTA_K = 128
NC = 4  # 1 KiB copies per wavefront and tile (K, and again V)
K0, V0, SUM0, KS0, LIST0, LDS0 = 0x10000000, 0x20000000, 0x30000000, 0x40000000, 0x50000000, 0


def generator():
    spec = importlib.util.spec_from_file_location("gen_dense_loop", CSRC / "gen_dense_loop.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def swizzled(row, chunk, rowbytes=128):
    """attention_kernel.hpp: byte offset of a 16-byte chunk of a row in a swizzled LDS tile."""
    chunks = rowbytes // 16
    return row * rowbytes + ((chunk ^ ((row // (256 // rowbytes)) & (chunks - 1))) << 4)


def k_source_offset(wave, i, lane):
    slot = (wave * NC + i) * 64 + lane
    row, phys = slot // 8, slot % 8
    return row * D + (phys ^ ((row // 2) & 7)) * 16


def v_source_offset(wave, i, lane, padded):
    slot = (wave * NC + i) * 64 + lane
    row, phys = slot // 8, slot % 8
    return row * padded + (phys ^ ((row // 2) & 7)) * 16


def interpret(program, operands, wave, padded, memory):
    """Runs the scalar side and the wait counters.  Returns (events, barriers); an event is
    (phase, kind, payload) with phase = barriers passed so far.  Asserts on the way that no
    instruction touches a register an LDS read or a scalar load is still to fill (LDS reads
    complete in order, scalar loads in any order, so with a scalar load in flight only a wait
    for zero proves anything)."""
    lines = [re.match(r'"(.*)\\n\\t"', line).group(1).split(";")[0].strip() for line in program.splitlines()]
    lines = [line for line in lines if line]
    labels = {line[:-1]: index for index, line in enumerate(lines) if line.endswith(":")}
    lanes = range(64)
    vreg = {
        246: [LDS0 + swizzled(l % 32, 0 + l // 32) for l in lanes], 247: [LDS0 + swizzled(l % 32, 2 + l // 32) for l in lanes],
        248: [LDS0 + swizzled(l % 32, 4 + l // 32) for l in lanes], 249: [LDS0 + swizzled(l % 32, 6 + l // 32) for l in lanes],
        250: [LDS0 + (l // 32) * 16 + 2048 for l in lanes],
        251: [k_source_offset(wave, 0, l) - (wave * NC) * 1024 for l in lanes],
        252: [k_source_offset(wave, 1, l) - (wave * NC + 1) * 1024 for l in lanes],
        253: [v_source_offset(wave, 0, l, padded) - (wave * NC) * 8 * padded for l in lanes],
        254: [v_source_offset(wave, 1, l, padded) - (wave * NC + 1) * 8 * padded for l in lanes],
    }
    sreg, state = {}, {"exec": (1 << 64) - 1, "scc": 0}
    lds_pending = []      # [(first register, registers)] oldest first
    scalar_pending = []   # [set of scalar registers]
    fragment = {}         # first register of a 4-register group -> lane addresses of the read that filled it

    def busy_vector():
        return {r for _, registers in lds_pending for r in registers}

    def busy_scalar():
        return {r for registers in scalar_pending for r in registers}

    def value(token):
        token = token.strip()
        if token in operands:
            return operands[token]
        if token == "exec":
            return state["exec"]
        pair = re.fullmatch(r"s\[(\d+):(\d+)\]", token)
        if pair:
            low = int(pair.group(1))
            assert not {low, low + 1} & busy_scalar(), token
            return sreg.get(low, 0) | (sreg.get(low + 1, 0) << 32)
        single = re.fullmatch(r"s(\d+)", token)
        if single:
            assert int(single.group(1)) not in busy_scalar(), token
            return sreg.get(int(single.group(1)), 0)
        if token == "m0":
            return sreg.get("m0", 0)
        return int(token, 0) & 0xFFFFFFFFFFFFFFFF

    def assign(token, result):
        token = token.strip()
        if token == "exec":
            state["exec"] = result & ((1 << 64) - 1)
        elif token == "m0":
            sreg["m0"] = result & 0xFFFFFFFF
        else:
            pair = re.fullmatch(r"s\[(\d+):(\d+)\]", token)
            if pair:
                low = int(pair.group(1))
                sreg[low], sreg[low + 1] = result & 0xFFFFFFFF, (result >> 32) & 0xFFFFFFFF
            else:
                sreg[int(token[1:])] = result & 0xFFFFFFFF

    def vector_registers(text):
        registers = {int(number) for number in re.findall(r"\bv(\d+)\b", text)}
        for low, high in re.findall(r"v\[(\d+):(\d+)\]", text):
            registers |= set(range(int(low), int(high) + 1))
        return registers

    events, barriers, pc, steps = [], 0, 0, 0
    while pc < len(lines):
        steps += 1
        assert steps < 5_000_000, "the loop does not end"
        line = lines[pc]
        pc += 1
        if line.endswith(":"):
            continue
        op, _, rest = line.partition(" ")
        args = [a.strip() for a in re.split(r",(?![^\[]*\])", rest)] if rest else []
        low32 = lambda token: value(token) & 0xFFFFFFFF
        if op.startswith(("v_", "ds_", "global_")):
            assert not vector_registers(rest) & busy_vector(), f"register still to be filled by an LDS read: {line}"
            for token in re.findall(r"\bs\d+\b|s\[\d+:\d+\]", rest):
                value(token)  # (asserts that no scalar load is still to fill it)
        if op == "s_barrier":
            assert not lds_pending and not scalar_pending
            barriers += 1
        elif op == "s_waitcnt":
            counter = re.search(r"lgkmcnt\((\d+)\)", rest)
            if counter:
                allowed = int(counter.group(1))
                if allowed == 0:
                    lds_pending, scalar_pending = [], []
                else:
                    assert not scalar_pending, f"a partial wait with a scalar load in flight: {line}"
                    lds_pending = lds_pending[len(lds_pending) - allowed:] if allowed < len(lds_pending) else lds_pending
            if "vmcnt" in rest:
                assert "vmcnt(0)" in rest
        elif op in ("s_mov_b32", "s_mov_b64"):
            assign(args[0], value(args[1]))
        elif op == "v_readfirstlane_b32":
            assign(args[0], vreg[int(args[1][1:])][0])
        elif op == "s_lshl_b32":
            assign(args[0], low32(args[1]) << low32(args[2]))
        elif op in ("s_add_u32", "s_addc_u32"):
            total = low32(args[1]) + low32(args[2]) + (state["scc"] if op == "s_addc_u32" else 0)
            state["scc"] = total >> 32
            assign(args[0], total)
        elif op in ("s_sub_u32", "s_subb_u32"):
            total = low32(args[1]) - low32(args[2]) - (state["scc"] if op == "s_subb_u32" else 0)
            state["scc"] = int(total < 0)
            assign(args[0], total)
        elif op == "s_min_u32":
            assign(args[0], min(low32(args[1]), low32(args[2])))
        elif op == "s_mul_i32":
            assign(args[0], low32(args[1]) * low32(args[2]))
        elif op == "s_mul_hi_u32":
            assign(args[0], (low32(args[1]) * low32(args[2])) >> 32)
        elif op == "s_cmp_eq_u32":
            state["scc"] = int(low32(args[0]) == low32(args[1]))
        elif op == "s_cmp_lg_u32":
            state["scc"] = int(low32(args[0]) != low32(args[1]))
        elif op == "s_cmp_lt_u32":
            state["scc"] = int(low32(args[0]) < low32(args[1]))
        elif op == "s_cselect_b32":
            assign(args[0], value(args[1]) if state["scc"] else value(args[2]))
        elif op == "s_cbranch_scc1":
            pc = labels[args[0]] if state["scc"] else pc
        elif op == "s_cbranch_vccz":
            pass  # the rescale block touches no memory; the GPU tests take both sides
        elif op in ("s_load_dword", "s_load_dwordx2", "s_load_dwordx4"):
            address = value(args[1]) + int(args[2], 0)
            events.append((barriers, "sload", address))
            count = {"s_load_dword": 1, "s_load_dwordx2": 2, "s_load_dwordx4": 4}[op]
            first = int(re.match(r"s\[?(\d+)", args[0]).group(1))
            for word in range(count):
                sreg[first + word] = memory.get(address + 4 * word, 0)
            scalar_pending.append(set(range(first, first + count)))
        elif op == "global_load_lds_dwordx4":
            assert "offset" not in args[1], "an instruction offset also moves the LDS address"
            base = value(args[1])
            register = int(args[0][1:])
            offsets = vreg[register]
            active = [l for l in lanes if (state["exec"] >> l) & 1]
            events.append((barriers, "copy", [(sreg["m0"] + 16 * l, base + offsets[l]) for l in active]))
        elif op == "ds_read_b128":
            match = re.fullmatch(r"v(\d+) offset:(\d+)", args[1])
            destination = int(re.match(r"v\[(\d+):", args[0]).group(1))
            addresses = [vreg[int(match.group(1))][l] + int(match.group(2)) for l in lanes]
            events.append((barriers, "read", (destination, addresses)))
            lds_pending.append((destination, set(range(destination, destination + 4))))
            fragment[destination] = tuple(addresses)
        elif op == "v_mfma_i32_32x32x32_i8":
            blocks = [re.match(r"v\[(\d+):", arg) for arg in args]
            start = int(blocks[3].group(1)) if blocks[3] else None
            events.append((barriers, "mfma", (int(blocks[0].group(1)), fragment[int(blocks[1].group(1))],
                                                int(blocks[2].group(1)), start)))
        elif op == "global_store_dwordx2":
            base, offsets = value(args[2]), vreg[int(args[0][1:])]
            active = [l for l in lanes if (state["exec"] >> l) & 1]
            events.append((barriers, "store", (int(re.match(r"v\[(\d+):", args[1]).group(1)), [base + offsets[l] for l in active])))
        elif op == "v_mbcnt_lo_u32_b32":
            assert args[1:] == ["-1", "0"]
            vreg[int(args[0][1:])] = [min(l, 32) for l in lanes]  # lanes below this one among the first 32
        elif op == "v_lshlrev_b32_e32" and int(args[2][1:]) in vreg:
            vreg[int(args[0][1:])] = [x << int(args[1]) for x in vreg[int(args[2][1:])]]
        elif op.startswith("v_"):
            for register in vector_registers(args[0]):
                fragment.pop(register, None)  # (a vector instruction rewrote it: no longer a fragment)
                if register < 246:
                    vreg.pop(register, None)  # (nor a lane index)
        elif op in ("s_nop", "s_setprio"):
            pass
        else:
            raise AssertionError(f"instruction the interpreter does not know: {line}")
    return events, barriers


def lane_halves():
    return [l // 32 for l in range(64)], [l % 32 for l in range(64)]


def k_fragment(stage, rb, kk):
    half, l32 = lane_halves()
    return tuple(stage * STAGE + swizzled(rb * 32 + l32[l], kk * 2 + half[l]) for l in range(64))


def v_fragment(stage, cb, rb):
    half, l32 = lane_halves()
    return tuple(stage * STAGE + 16384 + swizzled(cb * 32 + l32[l], rb * 2 + half[l]) for l in range(64))


S_BLOCK, ACC_BLOCK, Q_BLOCK, VF_BLOCK, PK_BLOCK = [0, 16, 32, 48], [64, 80, 96, 112], [192, 196, 200, 204], [208, 212, 216, 220], [224, 228]


def expected_reads(stage):
    """LDS reads of the tile in `stage`: K fragments into the accumulator registers, the
    accumulator seeds of channel block kk over the fragments of k-step kk, V fragments."""
    half, _ = lane_halves()
    reads = []
    for kk in range(4):
        for rb in range(4):
            reads.append((ACC_BLOCK[kk] + rb * 4, list(k_fragment(stage, rb, kk))))
        for b4 in range(4):
            reads.append((ACC_BLOCK[kk] + b4 * 4, [stage * STAGE + 32768 + (kk * 32 + b4 * 8 + half[l] * 4) * 4 for l in range(64)]))
    for rb in range(4):
        for cb in range(4):
            reads.append((VF_BLOCK[cb], list(v_fragment(stage, cb, rb))))
    return reads


def expected_matrix_instructions(stage):
    """Per destination block, in program order: (destination, lane addresses of the A fragment,
    first B register, first C register).  Score products start from the seed block that borrows
    the V fragment registers; value products accumulate over the seeds read from LDS."""
    chains = {}
    for rb in range(4):
        chains[S_BLOCK[rb]] = [(S_BLOCK[rb], k_fragment(stage, rb, kk), Q_BLOCK[kk], VF_BLOCK[0] if kk == 0 else S_BLOCK[rb])
                               for kk in range(4)]
    for cb in range(4):
        chains[ACC_BLOCK[cb]] = [(ACC_BLOCK[cb], v_fragment(stage, cb, rb), PK_BLOCK[rb & 1], ACC_BLOCK[cb]) for rb in range(4)]
    return chains


def test_generated_text_is_committed():
    gen = generator()
    assert {stem for _, _, stem in gen.PROGRAMS} == {path.name[:-4] for path in CSRC.glob("*_loop_d128.inc")}
    for sparse, capture, stem in gen.PROGRAMS:
        check_committed(gen, sparse, capture, stem)


def check_committed(gen, sparse, capture, stem):
    args = gen.parse([])
    args.sparse, args.capture = sparse, capture
    program, clobbers = gen.render(args)
    assert (CSRC / f"{stem}.inc").read_text() == program
    assert (CSRC / f"{stem}_clobbers.inc").read_text() == clobbers
    assert '"v255"' not in clobbers and '"v254"' not in clobbers  # the compiler's own register; an operand
    assert "s_store" not in program and "s_dcache" not in program and "s_atomic" not in program


STATS0, TILE_BYTES, STORING = 0x60000000, 40064 * 8, (1 << 20) - 1  # capture: rows of tile 0, bytes per tile, lanes that store


@pytest.mark.parametrize("program_kind", ["dense", "sparse", "capture"])
@pytest.mark.parametrize("tiles,padded", [(2, 256), (3, 384), (6, 1024), (9, 40064), (64, 8192)])
def test_memory_accesses_match_the_compiled_loop(program_kind, tiles, padded):
    """`tiles` listed tiles: the loop walks all but the last and copies in every one of them the
    next; every matrix instruction multiplies the fragment the compiled loop multiplies there; the
    capturing program stores eight bytes per storing lane and tile, tile-major."""
    gen = generator()
    args = gen.parse([])
    sparse, capture = program_kind == "sparse", program_kind == "capture"
    args.sparse, args.capture = sparse, capture
    program, _ = gen.render(args)
    key_tiles = padded // CTA_K
    listed = sorted(random.Random(tiles).sample(range(key_tiles), tiles)) if sparse else list(range(tiles))
    memory = {LIST0 + 4 * i: tile for i, tile in enumerate(listed)}
    for wave in range(4):
        operands = {"%[kptr]": K0 if sparse else K0 + CTA_K * D, "%[vptr]": V0 if sparse else V0 + CTA_K,
                    "%[sumptr]": SUM0 if sparse else SUM0 + D * 4, "%[ksptr]": KS0, "%[count]": tiles - 1,
                    "%[wave]": wave, "%[qs2]": 0x3F800000, "%[padded]": padded, "%[list]": LIST0,
                    "%[stats]": STATS0, "%[qlen8]": TILE_BYTES, "%[capexec]": STORING}
        events, barriers = interpret(program, operands, wave, padded, memory)
        assert barriers == tiles - 1

        def of(phase, kind):
            return [event[2] for event in events if event[0] == phase and event[1] == kind]

        assert of(0, "sload") == ([LIST0, KS0 + 16 * listed[0]] if sparse else [KS0])
        assert not of(0, "copy") and not of(0, "read") and not of(0, "mfma")
        for index in range(tiles - 1):
            phase, stage, other, following = index + 1, index & 1, (index & 1) ^ 1, listed[index + 1]
            wanted = []
            for i in range(NC):
                for lane in range(64):
                    wanted.append((other * STAGE + (wave * NC + i) * 1024 + 16 * lane,
                                   K0 + following * CTA_K * D + k_source_offset(wave, i, lane)))
                    wanted.append((other * STAGE + 16384 + (wave * NC + i) * 1024 + 16 * lane,
                                   V0 + following * CTA_K + v_source_offset(wave, i, lane, padded)))
            if wave == 0:  # accumulator seeds: 512 bytes by the first 32 lanes of wavefront 0
                wanted += [(other * STAGE + 32768 + 16 * lane, SUM0 + following * D * 4 + 16 * lane) for lane in range(32)]
            assert sorted(pair for copy in of(phase, "copy") for pair in copy) == sorted(wanted), (wave, index)
            assert sorted(of(phase, "read")) == sorted(expected_reads(stage)), (wave, index)
            issued = of(phase, "mfma")
            assert len(issued) == 32
            for destination, chain in expected_matrix_instructions(stage).items():
                assert [m for m in issued if m[0] == destination] == chain, (wave, index, destination)
            if sparse:
                assert of(phase, "sload") == [KS0 + 16 * following, LIST0 + 4 * min(index + 2, tiles - 1)], (wave, index)
            else:
                assert of(phase, "sload") == [KS0 + 16 * following], (wave, index)
        # statistics stores (row sum and tile maximum in two consecutive registers, by the storing
        # lanes only): the one of tile t at the top of tile t+1, none of the lanes before the first
        # tile, the last one behind the loop
        stores = [event[2] for event in events if event[1] == "store"]
        if capture:
            assert stores == [(234, [])] + [(234, [STATS0 + index * TILE_BYTES + 8 * lane for lane in range(20)])
                                            for index in range(tiles - 1)], wave
            phases = [event[0] for event in events if event[1] == "store"]
            assert phases == list(range(1, tiles)) + [tiles - 1]
        else:
            assert not stores


def test_wait_states_after_matrix_instructions():
    """No vector instruction touches a block an MFMA has written within 12 wait states of it
    (the distance gfx950 asks for after an 8-pass matrix instruction), counted as the assembler
    counts them: one per instruction, s_nop n counting n + 1."""
    gen = generator()
    for sparse, capture, _ in gen.PROGRAMS:
        args = gen.parse([])
        args.sparse, args.capture = sparse, capture
        lines = [re.match(r'"(.*)\\n\\t"', line).group(1).strip() for line in gen.render(args)[0].splitlines()]
        clock, written = 0, {}
        for line in lines:
            if not line or line.startswith(";") or line.endswith(":"):
                continue
            op = line.split()[0]
            if op == "s_barrier":  # (a new tile: everything issued before it is long done)
                written.clear()
            registers = [int(number) for number in re.findall(r"v(\d+)\b", line)]
            registers += [r for low, high in re.findall(r"v\[(\d+):(\d+)\]", line) for r in range(int(low), int(high) + 1)]
            if op.startswith("v_mfma"):
                destination = int(re.search(r"v\[(\d+):", line).group(1))
                for register in range(destination, destination + 16):
                    written[register] = clock
            elif op.startswith("v_") or op.startswith("ds_") or op.startswith("global_"):
                for register in registers:
                    assert clock - written.get(register, -100) >= 12 or register not in written, (line, register)
                    written.pop(register, None)
            clock += int(line.split()[1]) + 1 if op == "s_nop" else 1
