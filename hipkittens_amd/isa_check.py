"""Wait states between instructions that the compiler does not provide around inline assembly.

The kernels issue their vector-memory and matrix instructions from inline assembly. The compiler
treats such a statement as opaque: it places what the statement needs in front of it (a scalar
register restored from a spill slot with v_readlane_b32, a uniform value made scalar with
v_readfirstlane_b32), schedules its own instructions around it, and does not apply its hazard rules to
what is inside. gfx950 has no interlock for four cases that matter here, and a fifth check covers the
scalar loads that the kernels issue from inline assembly and wait for later:

* a scalar register written by a vector-ALU instruction and read by a vector-memory instruction
  (descriptor, scalar offset or base address) needs five wait states in between; with fewer the
  memory instruction may see the register's previous value: a load from a wild address;
* M0 written by a scalar instruction and read by a global->LDS load needs one wait state;
* the result registers of a matrix instruction of N passes (one pass = four clocks = one wait state)
  must not be read or written by any other kind of instruction, nor read as the A / B / scale operand
  of a matrix instruction, for N + 4 wait states after it issues (the distance the compiler keeps
  behind a matrix instruction it knows: 12 for the 8-pass FP8 one). A matrix instruction that
  follows another waits until the pipe has taken the one before it (N wait states after that one
  issued); that wait counts;
* the data registers of a vector-memory store of more than 64 bits must not be written by a vector-ALU
  instruction for two wait states after the store;
* the destination of a scalar load must not be touched before an `s_waitcnt lgkmcnt(0)` (scalar loads
  return out of order): the compiler takes the destination of an inline-assembly statement for
  written when the statement ends and is free to copy it to a spill slot at once.

`python -m hipkittens_amd.isa_check` compiles every csrc/*.hip to device assembly with the build's
flags and reports each place that some path through a kernel's code reaches with fewer wait states
than that (a taken branch counts as one wait state, like any instruction). A kernel that spills
scalar registers is the usual source of the first: the restore lands directly in front of the
statement that uses the register. The fix is an `s_nop` at the head of that statement, or fewer live
scalar values. It also reports any kernel that keeps registers in scratch memory (the compiler's
spill traffic would sit uncounted among the loads that the kernels wait for by count), and
`--resources` prints every kernel's register, spill, scratch and LDS figures.
"""
from __future__ import annotations

import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass, field
from pathlib import Path

from . import build as _build

VALU_SGPR_TO_VMEM = 5
M0_TO_LDS_DMA = 1
WIDE_STORE_TO_VALU_WRITE = 2
MFMA_RESULT_EXTRA = 4   # wait states beyond the instruction's passes (what the compiler leaves behind its own)

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
_WIDE_STORE = re.compile(r"(buffer|global|flat|scratch)_store_(dwordx[34]|format_xyzw?|format_d16_xyzw)")
_HORIZON = 32   # wait states after which a scalar write is forgotten (longer than any rule)


@dataclass
class Finding:
    function: str
    line: int
    instruction: str
    register: str
    wait_states: int
    needed: int

    def __str__(self) -> str:
        return (f"{self.function}: line {self.line}: {self.instruction} touches {self.register} "
                f"{self.wait_states} wait states after it was written (needs {self.needed})")


def _sgprs(token: str) -> list[int]:
    token = token.strip()
    m = re.fullmatch(r"s\[(\d+):(\d+)\]", token)
    if m:
        return list(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"s(\d+)", token)
    return [int(m.group(1))] if m else []


def _vector_registers(token: str) -> list[str]:
    """Vector and accumulation registers named by an operand: 'v[4:5]' -> ['v4', 'v5']."""
    token = token.strip()
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", token)
    if m:
        return [f"{m.group(1)}{i}" for i in range(int(m.group(2)), int(m.group(3)) + 1)]
    return [token] if re.fullmatch(r"[va]\d+", token) else []


def mfma_passes(op: str, args: str) -> int:
    """Passes of a matrix instruction (16 for one this table does not know: the longest there is)."""
    if "16x16x128_f8f6f4" in op:   # 8 passes with an fp8 operand, 4 when both are fp6 / fp4
        fmt = [int(m.group(1)) if m else 0 for m in (re.search(r"cbsz:(\d)", args), re.search(r"blgp:(\d)", args))]
        return 4 if min(fmt) >= 2 else 8
    if "16x16x32_bf16" in op or "16x16x32_f16" in op:
        return 4
    return 16


def _instruction(line: str):
    parts = line.split(None, 1)
    op, args = parts[0], parts[1] if len(parts) > 1 else ""
    operands = [t.strip() for t in re.split(r",(?![^\[]*\])", args)]
    return op, args, operands


@dataclass
class _State:
    since: dict = field(default_factory=dict)    # scalar register (or "m0") -> wait states since the write in question
    pending: dict = field(default_factory=dict)  # vector register -> (wait states still needed, out of)
    pipe: int = 0                                # wait states until the matrix pipe takes another instruction
    stored: dict = field(default_factory=dict)   # data register of a wide store -> wait states since the store
    loading: set = field(default_factory=set)    # scalar registers a scalar load may not have written yet

    def copy(self) -> "_State":
        return _State(dict(self.since), dict(self.pending), self.pipe, dict(self.stored), set(self.loading))

    def advance(self, states: int) -> None:
        for key in list(self.since):
            self.since[key] += states
            if self.since[key] >= _HORIZON:
                del self.since[key]
        for key in list(self.pending):
            left, total = self.pending[key]
            if left <= states:
                del self.pending[key]
            else:
                self.pending[key] = (left - states, total)
        self.pipe = max(0, self.pipe - states)
        for key in list(self.stored):
            self.stored[key] += states
            if self.stored[key] >= WIDE_STORE_TO_VALU_WRITE:
                del self.stored[key]

    def merge(self, other: "_State") -> "_State":
        """The least favourable of two states (two ways to reach the same place)."""
        out = self.copy()
        for key, value in other.since.items():
            out.since[key] = min(out.since.get(key, _HORIZON), value)
        for key, value in other.pending.items():
            out.pending[key] = max(out.pending.get(key, (0, 0)), value)
        out.pipe = min(out.pipe, other.pipe)
        for key, value in other.stored.items():
            out.stored[key] = min(out.stored.get(key, _HORIZON), value)
        out.loading |= other.loading
        return out

    def __eq__(self, other) -> bool:
        return ((self.since, self.pending, self.pipe, self.stored, self.loading) ==
                (other.since, other.pending, other.pipe, other.stored, other.loading))


def _step(state: _State, instr, function: str, findings: list | None) -> None:
    """Advances `state` over one instruction; reports into `findings`."""
    number, op, args, operands = instr

    def touches(operand_list):
        for operand in operand_list:
            for word in operand.split():
                for reg in _vector_registers(word):
                    if reg in state.pending and findings is not None:
                        left, total = state.pending[reg]
                        findings.append(Finding(function, number, op, reg, total - left, total))

    if op == "s_waitcnt":
        if re.search(r"lgkmcnt\(0\)", args):
            state.loading.clear()
    else:
        scalar_load = op.startswith(("s_load_", "s_buffer_load_"))
        if state.loading and findings is not None:
            for operand in (operands[1:] if scalar_load else operands):
                for word in operand.split():
                    for reg in _sgprs(word):
                        if reg in state.loading:
                            findings.append(Finding(function, number, op, f"s{reg} (scalar load in flight)", 0, 0))
        if scalar_load and operands:
            state.loading.update(_sgprs(operands[0]))
    if op.startswith("v_mfma"):
        touches(operands[1:3] + operands[4:6])   # A, B and scale operands (C chains on its own result)
        state.advance(state.pipe)                # waits for the pipe
        state.advance(1)
        passes = mfma_passes(op, args)
        state.pipe = passes - 1
        for reg in _vector_registers(operands[0]):
            state.pending[reg] = (passes + MFMA_RESULT_EXTRA, passes + MFMA_RESULT_EXTRA)
        return
    touches(operands)
    if op.startswith(_VMEM):
        for operand in operands:
            for word in operand.split():
                for reg in _sgprs(word):
                    if state.since.get(reg, _HORIZON) < VALU_SGPR_TO_VMEM and findings is not None:
                        findings.append(Finding(function, number, op, f"s{reg}", state.since[reg], VALU_SGPR_TO_VMEM))
        if re.search(r"\blds\b", args) and state.since.get("m0", _HORIZON) < M0_TO_LDS_DMA and findings is not None:
            findings.append(Finding(function, number, op, "m0", state.since["m0"], M0_TO_LDS_DMA))
    if op.startswith("v_") and operands and findings is not None:
        for reg in _vector_registers(operands[0]):
            if reg in state.stored:
                findings.append(Finding(function, number, op, reg, state.stored[reg], WIDE_STORE_TO_VALU_WRITE))
    state.advance(int(args.strip(), 0) + 1 if op == "s_nop" else 1)
    if _WIDE_STORE.match(op):
        data = operands[1] if op.startswith(("global_", "flat_", "scratch_")) else operands[0]
        for reg in _vector_registers(data):
            state.stored[reg] = 0
    if op.startswith("v_") and operands:
        written = _sgprs(operands[0])
        if len(operands) > 1 and _VALU_SECOND_DST.match(op):
            written += _sgprs(operands[1])
        for reg in written:
            state.since[reg] = 0
    elif op.startswith(_SALU_WRITERS) and operands:
        if operands[0] == "m0":
            state.since["m0"] = 0
        for reg in _sgprs(operands[0]):
            state.since.pop(reg, None)   # now a scalar-ALU result: no hazard towards vector memory


def _scan_function(function: str, blocks: list) -> list[Finding]:
    """blocks: [label or None, [instructions]] in layout order. The state at the head of a block is the
    least favourable over the ends of its predecessors (fall-through and branches that name its label)."""
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
    heads: list[_State | None] = [None] * len(blocks)
    heads[0] = _State()
    work = [0]
    while work:
        i = work.pop()
        state = heads[i].copy()
        for instr in blocks[i][1]:
            _step(state, instr, function, None)
        for j in successors[i]:
            merged = state.copy() if heads[j] is None else heads[j].merge(state)
            if heads[j] is None or merged != heads[j]:
                heads[j] = merged
                work.append(j)
    findings: list[Finding] = []
    for i, (_, instrs) in enumerate(blocks):
        if heads[i] is None:
            continue   # not reachable
        state = heads[i].copy()
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


def kernel_resources(asm_text: str) -> dict[str, dict[str, int]]:
    """Per kernel, from the metadata at the end of a `hipcc -S` file: register counts, spill counts,
    bytes of scratch (private segment) and of static LDS."""
    out: dict[str, dict[str, int]] = {}
    entry: dict[str, int] = {}
    name = None
    keys = {".agpr_count": "agprs", ".vgpr_count": "vgprs", ".sgpr_count": "sgprs",
            ".sgpr_spill_count": "sgpr_spills", ".vgpr_spill_count": "vgpr_spills",
            ".private_segment_fixed_size": "scratch_bytes", ".group_segment_fixed_size": "lds_bytes"}

    def flush():
        if name is not None:
            out[name] = entry

    for raw in asm_text.split("\n"):
        line = raw.strip()
        if raw.startswith("  - ."):         # first key of the next kernel's record (argument records sit deeper)
            flush()
            entry, name = {}, None
            line = line[2:]
        m = re.match(r"(\.\w+):\s+(\S+)$", line)
        if not m:
            continue
        if m.group(1) == ".name":
            name = m.group(2)
        elif m.group(1) in keys:
            entry[keys[m.group(1)]] = int(m.group(2))
    flush()
    return out


def memory_spills(asm_text: str) -> list[Finding]:
    """Kernels that keep registers in scratch memory. The compiler's spill stores and reloads are
    vector-memory operations of their own: they would sit, uncounted, between the loads whose
    completion the kernels track with hand-counted `s_waitcnt vmcnt(N)`."""
    findings = []
    for name, res in kernel_resources(asm_text).items():
        if res.get("scratch_bytes", 0) or res.get("vgpr_spills", 0):
            findings.append(Finding(name, 0, "kernel", "scratch memory", res.get("scratch_bytes", 0), 0))
    return findings


def device_assembly(src: Path, out: Path) -> None:
    cmd = [_build._hipcc(), *_build.HIPCC_FLAGS, *_build.PER_FILE_FLAGS.get(src.name, []),
           "--cuda-device-only", "-S", str(src), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src.name}:\n{res.stderr}")


def assembly_of_sources(sources: list[Path] | None = None, jobs: int = 8) -> dict[str, str]:
    """Device assembly of the sources (default: every .hip file under csrc/), by source file name."""
    sources = sources or sorted((_build.PKG_DIR / "csrc").rglob("*.hip"))
    with tempfile.TemporaryDirectory() as tmp:
        outs = [Path(tmp) / (s.stem + ".s") for s in sources]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(device_assembly, sources, outs))
        return {s.name: out.read_text() for s, out in zip(sources, outs)}


def check_texts(texts: dict[str, str]) -> list[Finding]:
    findings: list[Finding] = []
    for text in texts.values():
        findings += scan(text) + memory_spills(text)
    return findings


def check_sources(sources: list[Path] | None = None, jobs: int = 8) -> list[Finding]:
    """Compiles the sources (default: every .hip file under csrc/) to device assembly and scans them."""
    return check_texts(assembly_of_sources(sources, jobs))


def main() -> int:
    if "--resources" in sys.argv[1:]:   # a table of every kernel's registers, spills, scratch and LDS
        with tempfile.TemporaryDirectory() as tmp:
            for src in sorted((_build.PKG_DIR / "csrc").rglob("*.hip")):
                out = Path(tmp) / (src.stem + ".s")
                device_assembly(src, out)
                for name, res in kernel_resources(out.read_text()).items():
                    print(src.name, name, " ".join(f"{k}={v}" for k, v in res.items()))
        return 0
    findings = check_sources()
    for f in findings:
        print(f)
    print(f"{len(findings)} finding(s)")
    return 1 if findings else 0


if __name__ == "__main__":
    sys.exit(main())
