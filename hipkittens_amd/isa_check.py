"""Wait states between instructions that the compiler does not provide around inline assembly.

The kernels issue their vector-memory instructions from inline assembly. The compiler treats such a
statement as opaque: it places what the statement needs in front of it (a scalar register restored
from a spill slot with v_readlane_b32, a uniform value made scalar with v_readfirstlane_b32) and does
not apply its own hazard rules to what is inside. gfx950 has no interlock for two cases that matter
here:

* a scalar register written by a vector-ALU instruction and read by a vector-memory instruction
  (descriptor, scalar offset or base address) needs five wait states in between; with fewer the
  memory instruction may see the register's previous value: a load from a wild address;
* M0 written by a scalar instruction and read by a global->LDS load needs one wait state.

`python -m hipkittens_amd.isa_check` compiles every csrc/*.hip to device assembly with the build's
flags and reports each place that some path through a kernel's code reaches with fewer wait states
than that (a taken branch counts as one wait state, like any instruction). A kernel that spills
scalar registers is the usual source: the restore lands directly in front of the statement that uses
the register. The fix is an `s_nop` at the head of that statement, or fewer live scalar values.
"""
from __future__ import annotations

import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass
from pathlib import Path

from . import build as _build

VALU_SGPR_TO_VMEM = 5
M0_TO_LDS_DMA = 1

_VMEM = ("buffer_", "global_", "flat_", "scratch_")
# scalar-ALU / scalar-load instructions whose first operand is a destination
_SALU_WRITERS = (
    "s_mov", "s_cmov", "s_add", "s_sub", "s_mul", "s_and", "s_or", "s_xor", "s_nand", "s_nor", "s_xnor",
    "s_lshl", "s_lshr", "s_ashr", "s_min", "s_max", "s_cselect", "s_bfe", "s_bfm", "s_not", "s_brev",
    "s_bcnt", "s_ff", "s_flbit", "s_sext", "s_abs", "s_pack", "s_load", "s_buffer_load", "s_getpc",
    "s_wqm", "s_quadmask", "s_bitset",
)
# vector-ALU instructions whose second operand is a scalar carry / flag destination in the 64-bit encoding
_VALU_SECOND_DST = re.compile(r"v_(add|sub|subrev|addc|subb|subbrev)_co_|v_mad_[ui]64_[ui]32|v_div_scale")


@dataclass
class Finding:
    function: str
    line: int
    instruction: str
    register: str
    wait_states: int
    needed: int

    def __str__(self) -> str:
        return (f"{self.function}: line {self.line}: {self.instruction} reads {self.register} "
                f"{self.wait_states} wait states after it was written (needs {self.needed})")


def _sgprs(token: str) -> list[int]:
    token = token.strip()
    m = re.fullmatch(r"s\[(\d+):(\d+)\]", token)
    if m:
        return list(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"s(\d+)", token)
    return [int(m.group(1))] if m else []


_HORIZON = 32   # wait states after which a write is forgotten (longer than any rule)


def _instruction(line: str):
    parts = line.split(None, 1)
    op, args = parts[0], parts[1] if len(parts) > 1 else ""
    operands = [t.strip() for t in re.split(r",(?![^\[]*\])", args)]
    return op, args, operands


def _step(state: dict, instr, function: str, findings: list | None) -> None:
    """Advances `state` (scalar register -> wait states since a vector-ALU instruction wrote it; "m0" ->
    wait states since a scalar instruction wrote M0) over one instruction; reports into `findings`."""
    number, op, args, operands = instr
    if op.startswith(_VMEM):
        for operand in operands:
            for word in operand.split():
                for reg in _sgprs(word):
                    if state.get(reg, _HORIZON) < VALU_SGPR_TO_VMEM and findings is not None:
                        findings.append(Finding(function, number, op, f"s{reg}", state[reg], VALU_SGPR_TO_VMEM))
        if re.search(r"\blds\b", args) and state.get("m0", _HORIZON) < M0_TO_LDS_DMA and findings is not None:
            findings.append(Finding(function, number, op, "m0", state["m0"], M0_TO_LDS_DMA))
    states = int(args.strip(), 0) + 1 if op == "s_nop" else 1
    for key in list(state):
        state[key] += states
        if state[key] >= _HORIZON:
            del state[key]
    if op.startswith("v_") and operands:
        written = _sgprs(operands[0])
        if len(operands) > 1 and _VALU_SECOND_DST.match(op):
            written += _sgprs(operands[1])
        for reg in written:
            state[reg] = 0
    elif op.startswith(_SALU_WRITERS) and operands:
        if operands[0] == "m0":
            state["m0"] = 0
        for reg in _sgprs(operands[0]):
            state.pop(reg, None)   # now a scalar-ALU result: no hazard towards vector memory


def _scan_function(function: str, blocks: list) -> list[Finding]:
    """blocks: [label or None, [instructions]] in layout order. The state at the head of a block is the
    minimum over the ends of its predecessors (fall-through and branches that name its label)."""
    index = {b[0]: i for i, b in enumerate(blocks) if b[0] is not None}
    successors = []
    for i, (_, instrs) in enumerate(blocks):
        succ, falls = [], True
        if instrs:
            _, op, args, _ = instrs[-1]
            if op.startswith("s_cbranch") or op == "s_branch":
                target = args.strip()
                if target in index:
                    succ.append(index[target])
                falls = op != "s_branch"
            elif op in ("s_endpgm", "s_setpc_b64"):
                falls = False
        if falls and i + 1 < len(blocks):
            succ.append(i + 1)
        successors.append(succ)
    heads: list[dict | None] = [None] * len(blocks)
    heads[0] = {}
    work = [0]
    while work:
        i = work.pop()
        state = dict(heads[i])
        for instr in blocks[i][1]:
            _step(state, instr, function, None)
        for j in successors[i]:
            merged = dict(heads[j]) if heads[j] is not None else None
            if merged is None:
                merged = dict(state)
            else:
                for key, value in state.items():
                    merged[key] = min(merged.get(key, _HORIZON), value)
            if merged != heads[j]:
                heads[j] = merged
                work.append(j)
    findings: list[Finding] = []
    for i, (_, instrs) in enumerate(blocks):
        if heads[i] is None:
            continue   # not reachable
        state = dict(heads[i])
        for instr in instrs:
            _step(state, instr, function, findings)
    return findings


def scan(asm_text: str) -> list[Finding]:
    """Findings in the text of one `hipcc -S` device assembly file."""
    findings: list[Finding] = []
    function, blocks = None, []
    def flush():
        if function is not None and blocks:
            findings.extend(_scan_function(function, blocks))
    for number, raw in enumerate(asm_text.split("\n"), 1):
        line = raw.split(";")[0].strip()
        if not line:
            continue
        label = re.match(r"^([.$\w]+):$", line)
        if label:
            name = label.group(1)
            if name.startswith((".L", "LBB")):
                if function is not None:
                    blocks.append([name, []])
            else:
                flush()
                function, blocks = name, [[None, []]]
            continue
        if line.startswith(".") or function is None:
            continue
        op, args, operands = _instruction(line)
        blocks[-1][1].append((number, op, args, operands))
        if op.startswith("s_cbranch") or op in ("s_branch", "s_endpgm", "s_setpc_b64"):
            blocks.append([None, []])
    flush()
    findings.sort(key=lambda f: (f.function, f.line))
    return findings


def device_assembly(src: Path, out: Path) -> None:
    cmd = [_build._hipcc(), *_build.HIPCC_FLAGS, *_build.PER_FILE_FLAGS.get(src.name, []),
           "--cuda-device-only", "-S", str(src), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src.name}:\n{res.stderr}")


def check_sources(sources: list[Path] | None = None, jobs: int = 8) -> list[Finding]:
    """Compiles the sources (default: every csrc/*.hip) to device assembly and scans them."""
    sources = sources or sorted((_build.PKG_DIR / "csrc").glob("*.hip"))
    with tempfile.TemporaryDirectory() as tmp:
        outs = [Path(tmp) / (s.stem + ".s") for s in sources]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(device_assembly, sources, outs))
        findings: list[Finding] = []
        for out in outs:
            findings += scan(out.read_text())
    return findings


def main() -> int:
    findings = check_sources()
    for f in findings:
        print(f)
    print(f"{len(findings)} finding(s)")
    return 1 if findings else 0


if __name__ == "__main__":
    sys.exit(main())
