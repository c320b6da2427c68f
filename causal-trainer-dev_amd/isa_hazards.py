"""Static check of the compiled kernels for one hazard the compiler does not cover.

On gfx9-family hardware a memory instruction that reads a scalar register needs 5 wait states
after a vector instruction wrote that register (v_readfirstlane, v_readlane, carries, compares).
hipcc inserts those wait states in its own code but not in front of an ``asm`` statement, so a
scalar base that the compiler materialises with v_readfirstlane directly before an inline-asm
load, store or global->LDS copy is read stale: the access goes to whatever address the register
pair held before. ``scan`` walks device assembly (``hipcc -S --cuda-device-only``) and reports
every memory instruction whose scalar operands were written by a vector instruction fewer than
5 wait states earlier. It also reports the second hazard of that kind: a store of more than 8 bytes
reads its data registers late, and a vector instruction that writes one of them within 2 wait
states of the store replaces the data on its way out. ``python -m causal_trainer_dev_amd.isa_hazards`` compiles every source of
the library and scans it; tests/test_isa_hazards.py runs the same on the CPU.
"""

from __future__ import annotations

import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

WAIT_STATES = 5
STORE_DATA_WAIT_STATES = 2
_WIDE_STORE = re.compile(r"^\s*(global|buffer|flat|scratch)_store_dwordx[34]\s+(.*)")
_VECTOR_ALU = re.compile(r"^\s*v_\w+\s+(.*)")
_MEMORY = re.compile(r"^\s*(global_|buffer_|flat_|scratch_)")
_VECTOR_WRITES_SCALAR = re.compile(
    r"^\s*(v_readfirstlane_b32|v_readlane_b32|v_cmp\w*|v_add_co\w*|v_sub_co\w*|v_subrev_co\w*|v_addc\w*|"
    r"v_subb\w*|v_div_scale\w*|v_mad_u64_u32|v_mad_i64_i32)\s+(.*)")
_LABEL = re.compile(r"^([A-Za-z_.$][\w.$]*):")


def _scalar_registers(text: str) -> set:
    found = set()
    for match in re.finditer(r"s\[(\d+):(\d+)\]", text):
        found.update(range(int(match.group(1)), int(match.group(2)) + 1))
    for match in re.finditer(r"(?<![\w\[])s(\d+)\b", text):
        found.add(int(match.group(1)))
    if "vcc" in text:
        found.add("vcc")
    return found


def _vector_registers(text: str) -> set:
    found = set()
    for match in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        found.update(range(int(match.group(1)), int(match.group(2)) + 1))
    for match in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        found.add(int(match.group(1)))
    return found


def _wait_states(line: str) -> int:
    match = re.match(r"\s*s_nop\s+(\d+)", line)
    return int(match.group(1)) + 1 if match else 1


def scan(assembly: str) -> list[str]:
    """One message per memory instruction that reads a freshly vector-written scalar register."""

    problems, window, kernel = [], [], "?"
    for number, line in enumerate(assembly.splitlines(), start=1):
        text = line.strip()
        label = _LABEL.match(text)
        if label:
            if not text.startswith(".L"):
                kernel, window = label.group(1), []
            continue
        if not text or text.startswith((";", ".")):
            continue
        if _MEMORY.match(line):
            operands = text.split(None, 1)[1] if " " in text else ""
            used = _scalar_registers(operands)
            elapsed = 0
            for earlier_number, earlier in reversed(window):
                write = _VECTOR_WRITES_SCALAR.match(earlier)
                if write and _scalar_registers(write.group(2).split(",")[0]) & used:
                    problems.append(f"{kernel}: line {number} '{text}' reads a scalar register that line "
                                    f"{earlier_number} '{earlier.strip()}' wrote {elapsed} wait states earlier")
                    break
                elapsed += _wait_states(earlier)
                if elapsed >= WAIT_STATES:
                    break
        alu = _VECTOR_ALU.match(line)
        if alu and not text.startswith("v_mfma"):
            written = _vector_registers(alu.group(1).split(",")[0])
            elapsed = 0
            for earlier_number, earlier in reversed(window):
                store = _WIDE_STORE.match(earlier)
                if store:
                    fields = [field.strip() for field in store.group(2).split(",")]
                    # global_store: vaddr, vdata, saddr; buffer_store: vdata first
                    data = fields[0] if store.group(1) == "buffer" else (fields[1] if len(fields) > 1 else "")
                    if _vector_registers(data) & written:
                        problems.append(f"{kernel}: line {number} '{text}' writes store data of line "
                                        f"{earlier_number} '{earlier.strip()}' after {elapsed} wait states")
                        break
                elapsed += _wait_states(earlier)
                if elapsed >= STORE_DATA_WAIT_STATES:
                    break
        window.append((number, line))
        if len(window) > 16:
            del window[0]
    return problems


def private_accumulators(assembly: str, kernel: str) -> list[str]:
    """Checks a kernel that keeps values in accumulation registers across inline-assembly
    statements without telling the compiler (attn_dkv_wide_kernel): outside those statements the
    compiler must not touch an accumulation register (it would, to park a spilled vector register
    there), and no spilled register may be reloaded between the kernel's first and last workgroup
    barrier, i.e. inside its item loop, where the wait for the reload also waits for every
    asynchronous copy in flight."""

    problems, inside, in_asm, found = [], False, False, False
    reloads, barriers = [], []
    for number, line in enumerate(assembly.splitlines(), 1):
        text = line.strip()
        label = re.match(r"([A-Za-z_][\w$]*):", text)
        if label:
            inside = kernel in label.group(1)
            found = found or inside
            continue
        if not inside:
            continue
        if "#ASMSTART" in text:
            in_asm = True
        elif "#ASMEND" in text:
            in_asm = False
        elif not in_asm and not text.startswith((";", ".")):
            if re.search(r"\ba\[?\d", text) or "accvgpr" in text:
                problems.append(f"{kernel}: line {number} '{text}' uses an accumulation register outside the assembly statements")
            if text.startswith("scratch_load"):
                reloads.append((number, text))
            if text.startswith("s_barrier"):
                barriers.append(number)
    for number, text in reloads:
        if barriers and barriers[0] < number < barriers[-1]:
            problems.append(f"{kernel}: line {number} '{text}' reloads a spilled register inside the item loop")
    if not found:
        problems.append(f"{kernel}: not found in the assembly")
    return problems


def private_registers(assembly: str, kernel: str, lowest: int, highest: int) -> list[str]:
    """Checks a kernel whose inline-assembly statements keep values in the vector registers
    v[lowest:highest] and in accumulation registers from one statement to the next without telling
    the compiler (the interleaved forward: score buffers, fragment ring, output accumulator):
    outside those statements the compiled code must not name any of them."""

    problems, inside, in_asm, found = [], False, False, False
    for number, line in enumerate(assembly.splitlines(), 1):
        text = line.strip()
        label = re.match(r"([A-Za-z_][\w$]*):", text)
        if label:
            inside = kernel in label.group(1)
            found = found or inside
            continue
        if not inside:
            continue
        if "#ASMSTART" in text:
            in_asm = True
        elif "#ASMEND" in text:
            in_asm = False
        elif not in_asm and not text.startswith((";", ".")):
            code = text.split(";")[0]
            if re.search(r"\ba\[?\d", code) or "accvgpr" in code:
                problems.append(f"{kernel}: line {number} '{text}' uses an accumulation register outside the assembly statements")
            if any(lowest <= register <= highest for register in _vector_registers(code)):
                problems.append(f"{kernel}: line {number} '{text}' uses a vector register of v[{lowest}:{highest}] "
                                "outside the assembly statements")
    if not found:
        problems.append(f"{kernel}: not found in the assembly")
    return problems


def block_mix(assembly: str, kernel: str) -> list[dict]:
    """Instruction mix of every basic block of `kernel` (the first function whose label contains the
    name): a list of {"label", "valu", "exp", "max3", "mfma", "salu", "lds", "vmem"} in program order.
    "valu" counts vector ALU instructions other than MFMA (v_exp and v_max3 included; they are also
    counted on their own). Used to hold the steady-state paths of the attention kernels to an
    instruction budget per MFMA."""

    blocks, inside, found = [], False, False
    current = None

    def start(label):
        nonlocal current
        current = {"label": label, "valu": 0, "exp": 0, "max3": 0, "mfma": 0, "salu": 0, "lds": 0, "vmem": 0}
        blocks.append(current)

    for line in assembly.splitlines():
        text = line.strip()
        fallthrough = re.match(r"; %bb\.(\d+):", text)
        if fallthrough and inside:
            start("%bb." + fallthrough.group(1))  # a block entered by falling through has no label of its own
            continue
        if not text or text.startswith((";", "//")):
            continue
        function = re.match(r"([A-Za-z_][\w$]*):", text)
        if function and not text.startswith(".L"):
            if found and inside:
                break                      # next function: done
            inside = kernel in function.group(1)
            if inside:
                found = True
                start("entry")
            continue
        if not inside:
            continue
        if text.startswith(".Lfunc_end"):
            break
        if re.match(r"\.LBB\w+:", text):
            start(text.split(":")[0])
            continue
        if text.startswith("."):
            continue
        op = text.split()[0]
        if op.startswith("v_mfma"):
            current["mfma"] += 1
        elif op.startswith("v_"):
            current["valu"] += 1
            if op.startswith("v_exp"):
                current["exp"] += 1
            if op.startswith("v_max3"):
                current["max3"] += 1
        elif op.startswith("ds_"):
            current["lds"] += 1
        elif op.startswith(("global_", "scratch_", "buffer_", "flat_")):
            current["vmem"] += 1
        elif op.startswith("s_"):
            current["salu"] += 1
    return blocks


def device_assembly(source: Path, flags) -> str:
    from . import build as recipe

    with tempfile.TemporaryDirectory() as scratch:
        target = Path(scratch) / (source.stem + ".s")
        command = [recipe.hipcc(), *[f for f in flags if f != "-fPIC"], "--cuda-device-only", "-S", str(source),
                   "-o", str(target)]
        done = subprocess.run(command, capture_output=True, text=True)
        if done.returncode != 0:
            raise RuntimeError(done.stderr)
        return target.read_text()


def scan_library() -> dict[str, list[str]]:
    """Compiles every source of the library to device assembly and scans it."""

    from . import build as recipe

    sources = [recipe.CSRC / name for name in recipe.SOURCES]
    with ThreadPoolExecutor(max_workers=4) as pool:
        texts = list(pool.map(lambda path: device_assembly(path, recipe.HIP_FLAGS), sources))
    findings = {path.name: scan(text) for path, text in zip(sources, texts)}
    for path, text in zip(sources, texts):
        if path.name == "ct_attn.hip":
            findings[path.name] += private_accumulators(text, "attn_dkv_wide_kernel")
            for heads in (1, 2, 4):
                findings[path.name] += private_registers(text, f"attn_fwd_kernelILi128ELi{heads}E", 112, 191)
    return findings


if __name__ == "__main__":
    findings = scan_library()
    for name, problems in findings.items():
        print(f"{name}: {len(problems)} hazard(s)")
        for problem in problems:
            print("  " + problem)
    sys.exit(1 if any(findings.values()) else 0)
