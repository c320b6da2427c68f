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
        self.unread = {}           # register -> index of the LDS read whose data no MFMA has used yet
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
                    self.problems.append(f"line {number} '{line}' overwrites a fragment no MFMA has read")
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
    return {
        "pv": gen.pv_sequence(4, 4), "qk": gen.qk_sequence(4, 4), "dq_sdp_half": gen.dq_sdp_half_sequence(),
        "dq_acc_half": gen.dq_acc_half_sequence(), "dkv_sdp": gen.dkv_sdp_sequence(), "dkv_acc": gen.dkv_acc_sequence(),
        "dkvw_step": gen.dkvw_step_sequence(), "dkvw_masked": gen.dkvw_step_sequence(masked=True),
        "dkvw_run": gen.dkvw_run_sequence(),
    }


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
    assert any("no MFMA has read" in p for p in Model().run(lost).problems)
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


def test_committed_include_is_what_the_generator_prints(gen):
    import subprocess
    import sys

    printed = subprocess.run([sys.executable, GENERATOR], capture_output=True, text=True, check=True).stdout
    with open(os.path.join(os.path.dirname(GENERATOR), "ct_attn_asm.inc")) as handle:
        assert handle.read() == printed
