"""Static checks of the hand-scheduled instruction streams that gen_attn_asm.py emits.

The streams name physical registers and count their own LDS reads in flight, so nothing but these
checks (and the GPU parity tests) stands between an edit of the generator and a silently wrong
kernel. An in-order model of one wavefront is enough: LDS reads complete in issue order, and
`s_waitcnt lgkmcnt(n)` returns when at most n are outstanding.
"""

import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GENERATOR = os.path.join(ROOT, "causal-trainer-dev_amd", "csrc", "gen_attn_asm.py")


@pytest.fixture(scope="module")
def gen():
    spec = importlib.util.spec_from_file_location("gen_attn_asm", GENERATOR)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def _registers(operand):
    """Fixed vector registers an operand text names (asm operands such as %3 name none)."""
    found = set()
    for lo, hi in re.findall(r"\bv\[(\d+):(\d+)\]", operand):
        found.update(range(int(lo), int(hi) + 1))
    for single in re.findall(r"\bv(\d+)\b", operand):
        found.add(int(single))
    return found


def _split(line):
    mnemonic, _, rest = line.partition(" ")
    operands = [part.strip() for part in rest.split(",")] if rest else []
    # v[a:b] contains no comma, offset:... rides on the last operand
    return mnemonic, operands


class Model:
    def __init__(self):
        self.pending = []          # (destination registers) of LDS reads in flight, in issue order
        self.unread = {}           # register -> index of the LDS read whose data nothing has used yet
        self.mfmas = 0
        self.last_mfma_write = {}  # register -> number of the MFMA that last wrote it
        self.problems = []

    def busy(self):
        return set().union(*self.pending) if self.pending else set()

    def run(self, lines):
        for number, line in enumerate(lines):
            mnemonic, ops = _split(line)
            if mnemonic.startswith("ds_read"):
                dest = _registers(ops[0])
                stale = [r for r in dest if r in self.unread]
                if stale:
                    self.problems.append(f"line {number} '{line}' overwrites LDS data nothing has read")
                if dest & self.busy():
                    self.problems.append(f"line {number} '{line}' writes registers of a read still in flight")
                self.pending.append(dest)
                for r in dest:
                    self.unread[r] = number
                if len(self.pending) > 15:
                    self.problems.append(f"line {number}: more than 15 LDS reads in flight")
            elif mnemonic == "s_waitcnt" and "lgkmcnt" in line:
                keep = int(re.search(r"lgkmcnt\((\d+)\)", line).group(1))
                while len(self.pending) > keep:
                    self.pending.pop(0)
            elif mnemonic.startswith("v_mfma"):
                sources = set().union(*[_registers(op) for op in ops[1:]])
                if sources & self.busy():
                    self.problems.append(f"line {number} '{line}' reads registers of an LDS read still in flight")
                for r in sources:
                    self.unread.pop(r, None)
                for r in _registers(ops[0]):
                    self.last_mfma_write[r] = self.mfmas
                    self.unread.pop(r, None)
                self.mfmas += 1
            elif mnemonic.startswith("v_"):
                sources = set().union(*[_registers(op) for op in ops[1:]]) if len(ops) > 1 else set()
                if sources & self.busy():
                    self.problems.append(f"line {number} '{line}' reads registers of an LDS read still in flight")
                for r in sources:
                    self.unread.pop(r, None)       # (ids read from LDS are consumed by compares)
                    written = self.last_mfma_write.get(r)
                    # an MFMA result is read by the vector ALU only after two more MFMAs have been
                    # issued: the producer has then left the matrix pipe
                    if written is not None and self.mfmas - written < 3:
                        self.problems.append(f"line {number} '{line}' reads v{r} {self.mfmas - written - 1} MFMA(s) "
                                             "after the MFMA that wrote it")
                for r in _registers(ops[0]):
                    self.last_mfma_write.pop(r, None)
                    self.unread.pop(r, None)
        return self


def _sequences(gen):
    sequences = {
        "pv": gen.pv_sequence(4, 4), "qk": gen.qk_sequence(4, 4), "dq_sdp_half": gen.dq_sdp_half_sequence(),
        "dq_acc_half": gen.dq_acc_half_sequence(), "dkv_sdp": gen.dkv_sdp_sequence(), "dkv_acc": gen.dkv_acc_sequence(),
        "dkvw_step": gen.dkvw_step_sequence(), "dkvw_masked": gen.dkvw_step_sequence(masked=True),
        "dkvw_run": gen.dkvw_run_sequence(),
    }
    for cur in ("a", "b"):
        for name, lines in gen.fwd_statements(cur).items():
            sequences["fwd_%s_%s" % (name.lower(), cur)] = lines
    return sequences


def test_fragment_rings_and_wait_counts(gen):
    for name, lines in _sequences(gen).items():
        model = Model().run(lines)
        assert model.problems == [], (name, model.problems[:5])
        assert not model.unread, (name, "fragments read from LDS and never used", sorted(model.unread)[:8])


def test_model_catches_the_mistakes_it_is_meant_for(gen):
    good = gen.qk_sequence(4, 4)
    assert Model().run(good).problems == []
    # a wait that lets one read too many stay in flight
    loose = list(good)
    first_wait = next(i for i, line in enumerate(loose) if "lgkmcnt(3)" in line)
    loose[first_wait] = "s_waitcnt lgkmcnt(4)"
    assert any("still in flight" in p for p in Model().run(loose).problems)
    # a fragment overwritten before its MFMA
    lost = [line for line in good]
    mfma = next(i for i, line in enumerate(lost) if line.startswith("v_mfma"))
    del lost[mfma]
    assert any("nothing has read" in p for p in Model().run(lost).problems)
    # arithmetic directly behind the MFMA that produces its input
    wide = gen.dkvw_step_sequence()
    s0 = gen.W_S[0]
    block = "v[%d:%d]" % (s0, s0 + 15)
    last_s0 = max(i for i, line in enumerate(wide) if line.startswith("v_mfma") and line.split()[1].startswith(block))
    early = wide[:last_s0 + 1] + ["v_mul_f32_e32 v%d, %%33, v%d" % (s0, s0)] + wide[last_s0 + 1:]
    assert any("after the MFMA that wrote it" in p for p in Model().run(early).problems)


def test_wide_stream_structure(gen):
    lines = gen.dkvw_step_sequence()
    mfmas = [line for line in lines if line.startswith("v_mfma")]
    assert len(mfmas) == 64
    # 16 accumulators, two k-steps each, every one a read-modify-write of the same registers
    per_accumulator = {}
    for line in mfmas[32:]:
        _, ops = _split(line)
        assert ops[0] == ops[3] and ops[0].startswith("a["), line
        per_accumulator[ops[0]] = per_accumulator.get(ops[0], 0) + 1
    assert len(per_accumulator) == 16 and set(per_accumulator.values()) == {2}
    # the packed P / dS fragments an accumulating MFMA reads were written after the block's last
    # S / dP MFMA and before this MFMA
    for kb, (s_base, dp_base) in enumerate(zip(gen.W_S, gen.W_DP)):
        for base in (s_base, dp_base):
            block = "v[%d:%d]" % (base, base + 15)
            last_product = max(i for i, line in enumerate(lines) if line.startswith("v_mfma") and _split(line)[1][0] == block)
            for step in range(2):
                operand = "v[%d:%d]" % (base + 4 * step, base + 4 * step + 3)
                readers = [i for i, line in enumerate(lines) if line.startswith("v_mfma") and _split(line)[1][1] == operand]
                assert len(readers) == 4, (operand, readers)
                for k in range(4 * step, 4 * step + 4):
                    packs = [i for i, line in enumerate(lines)
                             if line.startswith("v_cvt_pk_bf16_f32 v%d," % (base + k))]
                    assert len(packs) == 1 and last_product < packs[0] < min(readers), (operand, k)
    # ten copies, each behind an MFMA that follows the write of m0
    copies = [i for i, line in enumerate(lines) if line.startswith("global_load_lds")]
    assert len(copies) == 10
    for i in copies:
        back = [line for line in lines[max(0, i - 4):i]]
        assert any(line.startswith("s_add_u32 m0") for line in back) and any(line.startswith("v_mfma") for line in back), lines[i]
    # the exec mask is narrowed around the two statistics copies only and restored right behind them
    narrowed = [i for i, line in enumerate(lines) if line == "s_mov_b64 exec, 0xff"]
    assert len(narrowed) == 2
    for i in narrowed:
        assert lines[i + 1].startswith("global_load_lds") and lines[i + 2] == "s_mov_b64 exec, -1"


def _vector_alu(lines):
    return [line for line in lines if line.startswith("v_") and not line.startswith("v_mfma")]


@pytest.mark.parametrize("cur", ["a", "b"])
def test_forward_interleaved_statements(gen, cur):
    """The forward's three statements per key tile: MFMA counts, how much vector work sits behind
    an MFMA, that the statements without MFMAs run the very same vector instructions (the two forms
    of a step must give the same bits), where the bf16 pairs go, and the copies."""

    statements = gen.fwd_statements(cur)
    s0, other = gen.FWD_S[cur], gen.FWD_S[gen.other(cur)]
    mfmas = {name: [line for line in lines if line.startswith("v_mfma")] for name, lines in statements.items()}
    assert [len(mfmas[name]) for name in ("MAX", "EXP_A", "EXP_B", "PV", "PV_LATE", "QK")] == [8, 8, 16, 16, 8, 16]
    # about five vector instructions fit behind an MFMA (microbenchmark): no statement asks for more
    for name in ("MAX", "EXP_A", "EXP_B"):
        assert len(_vector_alu(statements[name])) / len(mfmas[name]) <= 5.0, name
    total = sum(len(_vector_alu(statements[name])) for name in ("MAX", "EXP_A", "EXP_B"))
    assert total / 32 <= 4.3, total

    # the same vector instructions with and without the MFMAs; for the exponentials, which the
    # interleaved form cuts into two statements (so the software pipeline drains once in between),
    # the same instructions per score and the same order of the additions into the sum
    assert _vector_alu(statements["MAX"]) == _vector_alu(statements["MAX_ONLY"])
    split = _vector_alu(statements["EXP_A"]) + _vector_alu(statements["EXP_B"])
    assert sorted(split) == sorted(_vector_alu(statements["EXP_ONLY"]))
    additions = lambda lines: [line for line in lines if line.startswith("v_add_f32")]
    assert additions(split) == additions(_vector_alu(statements["EXP_ONLY"]))
    # the products of the two forms are the same MFMAs in the same order
    assert mfmas["MAX"] + mfmas["EXP_A"] == mfmas["PV"] and mfmas["EXP_A"] == mfmas["PV_LATE"]
    assert mfmas["EXP_B"] == mfmas["QK"]

    for exponent in (_vector_alu(statements["EXP_ONLY"]), split):
        # nothing reads the result of a transcendental instruction directly behind it
        for before, after in zip(exponent, exponent[1:]):
            if before.startswith("v_exp_f32"):
                written = _registers(_split(before)[1][0])
                assert not written & set().union(*[_registers(op) for op in _split(after)[1][1:]]), (before, after)
        # the sum runs in score order; score i: fma, exp2, add, and its pair's packing, in that order
        adds = [line for line in exponent if line.startswith("v_add_f32")]
        assert [_split(line)[1][2] for line in adds] == ["v%d" % (s0 + i) for i in range(32)]
        position = {line: index for index, line in enumerate(exponent)}
        pack_of = lambda pair: position["v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (s0 + pair, s0 + 2 * pair, s0 + 2 * pair + 1)]
        for i in range(32):
            register = s0 + i
            fma = position["v_fma_f32 v%d, v%d, %%[c], -%%[m]" % (register, register)]
            exp2 = position["v_exp_f32_e32 v%d, v%d" % (register, register)]
            add = position["v_add_f32_e32 %%[psum], %%[psum], v%d" % register]
            assert fma < exp2 < add < pack_of(i // 2), i
            # the pair's packing overwrites score i // 2, whose own packing (pair i // 4) is done
            assert pack_of(i // 4) <= pack_of(i // 2), i
        assert sum(line.startswith("v_cvt_pk_bf16_f32") for line in exponent) == 16

    # P^T of the tile before: the first 16 registers of the other buffer, k-step by k-step; the
    # next tile's scores go to the other buffer and only the last statement writes there
    for index, line in enumerate(mfmas["PV"]):
        step = index // 4
        assert _split(line)[1][2] == "v[%d:%d]" % (other + 4 * step, other + 4 * step + 3), line
        assert _split(line)[1][0] == _split(line)[1][3] == "a[%d:%d]" % (16 * (index % 4), 16 * (index % 4) + 15)
    for index, line in enumerate(mfmas["QK"]):
        block = index % 2
        assert _split(line)[1][0] == "v[%d:%d]" % (other + 16 * block, other + 16 * block + 15), line
    for name in ("MAX", "EXP_A", "MAX_ONLY", "EXP_ONLY", "MASK_CAUSAL", "MASK_IDS"):
        for line in statements[name]:
            if line.startswith(("v_", "ds_read")):
                destination = _registers(_split(line)[1][0])
                assert not destination & set(range(other, other + 32)), (name, line)
    # no statement names a register outside the private window (and its operands)
    for name, lines in statements.items():
        for line in lines:
            named = set().union(*[_registers(op) for op in _split(line)[1]]) if " " in line else set()
            assert all(gen.FWD_FIRST_PRIVATE <= r <= gen.FWD_LAST_PRIVATE for r in named), (name, line)

    # the step's four copies ride in the first statement: V pieces, then K pieces, each with m0 set
    # at least one instruction ahead and nothing else touching m0 in between
    first = statements["MAX"]
    copies = [i for i, line in enumerate(first) if line.startswith("global_load_lds")]
    assert [first[i] for i in copies] == ["global_load_lds_dwordx4 %%[off%d], %%[%s]" % (g % 2, "vsrc" if g < 2 else "ksrc")
                                          for g in range(4)]
    settings = [i for i, line in enumerate(first) if line.startswith("s_mov_b32 m0")]
    assert [first[i] for i in settings] == ["s_mov_b32 m0, %%[d%d]" % g for g in range(4)]
    for g in range(4):
        assert settings[g] + 1 < copies[g] and (g == 3 or copies[g] < settings[g + 1])
    for name in ("EXP_A", "EXP_B", "PV", "PV_LATE", "QK"):
        assert not any("m0" in line or line.startswith("global_") for line in statements[name]), name


def test_forward_masks(gen):
    """The mask statements: one compare and one select per score, the key offset of a score register
    as the accumulator layout has it (block 32 kb, then 8 (r / 4) + r % 4, plus 4 for the lanes of
    the upper half)."""

    for cur in ("a", "b"):
        s0 = gen.FWD_S[cur]
        causal = gen.fwd_statements(cur)["MASK_CAUSAL"]
        assert len(causal) == 64
        for i in range(32):
            offset = 32 * (i // 16) + 8 * ((i % 16) // 4) + (i % 16) % 4
            assert causal[2 * i] == "v_cmp_le_i32_e32 vcc, %d, %%[rel]" % offset
            assert causal[2 * i + 1] == "v_cndmask_b32_e32 v%d, %%[ninf], v%d, vcc" % (s0 + i, s0 + i)
        # ids: run the statement on a model of the id ring (key k's id at byte 4 k; the lane's pointer
        # is the address of key 4 * half): every score must be compared with the id of its own key,
        # and no register may be read before the wait that covers its load
        for half in (0, 1):
            registers, landed, in_flight = {}, set(), []
            compared = {}
            pending_compare = None
            for line in gen.fwd_statements(cur)["MASK_IDS"]:
                name, operands = _split(line)
                if name == "s_waitcnt":
                    allowed = int(operands[0][len("lgkmcnt("):-1])
                    while len(in_flight) > allowed:
                        landed |= in_flight.pop(0)
                elif name == "ds_read_b128":
                    offset = int(operands[2][len("offset:"):]) if len(operands) > 2 else int(line.split("offset:")[1])
                    quad = sorted(_registers(operands[0]))
                    assert len(quad) == 4 and offset % 16 == 0
                    for e, register in enumerate(quad):
                        registers[register] = 4 * half + offset // 4 + e     # the key whose id it holds
                    landed -= set(quad)
                    in_flight.append(set(quad))
                elif name == "v_cmp_eq_u32_e32":
                    assert operands[:2] == ["vcc", "%[segq]"]
                    (register,) = _registers(operands[2])
                    assert register in landed, line
                    pending_compare = registers[register]
                elif name == "v_cndmask_b32_e32":
                    (score,) = _registers(operands[0])
                    assert operands[1] == "%[ninf]" and _registers(operands[2]) == {score} and operands[3] == "vcc"
                    compared[score - s0] = pending_compare
                    pending_compare = None
                else:
                    raise AssertionError(line)
            assert compared == {i: 32 * (i // 16) + 8 * ((i % 16) // 4) + (i % 16) % 4 + 4 * half for i in range(32)}


def test_committed_include_is_what_the_generator_prints(gen):
    import subprocess
    import sys

    printed = subprocess.run([sys.executable, GENERATOR], capture_output=True, text=True, check=True).stdout
    with open(os.path.join(os.path.dirname(GENERATOR), "ct_attn_asm.inc")) as handle:
        assert handle.read() == printed
