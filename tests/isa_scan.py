"""A reader of the gfx950 assembly that hipcc makes of this library's kernels: does any
instruction use the result registers of a matrix instruction sooner than the hardware
allows?

CDNA matrix instructions write their result some cycles after they issue, and the hardware
does not hold back a vector instruction that reads or overwrites those registers earlier:
the compiler has to keep ``WAIT_STATES`` other instructions (or ``s_nop``) in between, on
every path.  It once did not: with a wave-uniform branch directly behind a
``v_mfma_f32_16x16x32_bf16`` whose target began by copying the accumulators back
(``v_accvgpr_read_b32``), the taken path had a branch and two instructions between the two,
and one of a lane's four sums lost its latest product.  This module finds such sequences
by following every path from each matrix instruction for ``WAIT_STATES`` wait states.
"""
import hashlib
import os
import re
import subprocess
import tempfile

# v_mfma_f32_16x16x32_bf16 on gfx950: what the compiler keeps between the instruction and a
# vector instruction that touches its result (a branch counts as one), read off its own
# output where nothing else could be scheduled in between
WAIT_STATES = 7

_REG = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")


def registers(text):
    out = set()
    for m in _REG.finditer(text):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(3), i) for i in range(int(m.group(4)), int(m.group(5)) + 1))
    return out


def kernels_of(assembly: str):
    """{kernel name: [("label", name) | ("ins", text)]} of an assembly file's text."""
    kernels, cur = {}, None
    for line in assembly.splitlines():
        m = re.match(r"^(_Z\w+|[A-Za-z_]\w*):", line)
        if m and not line.startswith(".L"):
            cur = kernels.setdefault(m.group(1), [])
            continue
        if cur is None:
            continue
        if line.startswith(".Lfunc_end"):
            cur = None
            continue
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            cur.append(("label", m.group(1)))
            continue
        t = line.split(";")[0].strip()
        if not t or t.startswith(".") or t.startswith("//"):
            continue
        cur.append(("ins", t))
    return {k: v for k, v in kernels.items() if any(kind == "ins" for kind, _ in v)}


def _is_matrix(op: str) -> bool:
    return op.startswith("v_mfma") or op.startswith("v_smfmac")


def early_uses(items, wait_states: int = WAIT_STATES):
    """[(matrix instruction, using instruction, wait states between)] for every use that
    comes too early on some path."""
    flat, label_at = [], {}
    for kind, val in items:
        if kind == "label":
            label_at[val] = len(flat)
        else:
            flat.append(val)
    bad = []
    for i, ins in enumerate(flat):
        if not _is_matrix(ins.split()[0]):
            continue
        dst = registers(ins.split(None, 1)[1].split(",")[0])
        seen = set()
        stack = [(i + 1, 0)]
        while stack:
            j, ws = stack.pop()
            while j < len(flat) and ws < wait_states:
                t = flat[j]
                op = t.split()[0]
                if op == "s_endpgm":
                    break
                if op.startswith("s_cbranch") or op == "s_branch":
                    target = t.split()[-1]
                    if target in label_at and (label_at[target], ws + 1) not in seen:
                        seen.add((label_at[target], ws + 1))
                        stack.append((label_at[target], ws + 1))
                    if op == "s_branch":
                        break
                    ws += 1
                    j += 1
                    continue
                operands = t.split(None, 1)[1] if " " in t else ""
                if _is_matrix(op):
                    # a matrix instruction that takes the result as its accumulator is held
                    # back by the hardware; one that overwrites it ends the window
                    if registers(operands.split(",")[0]) & dst:
                        break
                elif op != "s_nop" and registers(operands) & dst:
                    bad.append((ins, t, ws))
                    break
                m = re.match(r"s_nop (\d+)", t)
                ws += int(m.group(1)) + 1 if m else 1
                j += 1
    return bad


def loads_touched_before_their_wait(assembly: str):
    """Loads that a kernel writes as inline asm are not known to the compiler as loads: it may
    use their registers as soon as the statement is over, while the data is still under way.
    The kernels therefore name those registers in the asm wait that follows (which orders
    every reader behind it).  This checks the result: between an asm ``global_load`` and the
    next asm ``s_waitcnt vmcnt`` in the kernel's text, no instruction may mention the load's
    registers.  Returns [(kernel, load, offending instruction)]."""
    out = []
    for chunk in re.split(r"\n(?=[A-Za-z_]\w*:)", assembly):
        m = re.match(r"([A-Za-z_]\w*):", chunk)
        if not m:
            continue
        lines = chunk.split("\n")
        for i, line in enumerate(lines):
            if "#ASMSTART" not in line or i + 1 >= len(lines) or "global_load" not in lines[i + 1]:
                continue
            load = lines[i + 1].strip()
            dst = registers(load.split(None, 1)[1].split(",")[0])
            j = i + 3                                      # behind the load's #ASMEND
            while j < len(lines):
                t = lines[j].split(";")[0].strip() if "#ASM" not in lines[j] else lines[j].strip()
                if "#ASMSTART" in t and j + 1 < len(lines) and "s_waitcnt" in lines[j + 1] \
                        and "vmcnt" in lines[j + 1]:
                    break
                if t.startswith("s_endpgm"):
                    out.append((m.group(1), load, "the kernel ends before a wait"))
                    break
                if t and not t.startswith(".") and "#ASM" not in t:
                    operands = t.split(None, 1)[1] if len(t.split(None, 1)) > 1 else ""
                    if registers(operands) & dst:
                        out.append((m.group(1), load, t))
                        break
                j += 1
    return out


def assembly_of(module: str) -> str:
    """The device assembly of csrc/<module>.hip with the library's own flags, compiled once
    per state of the sources into the temporary directory."""
    from gpt_fast_amd.csrc import build as B
    flags = [f for f in B.FLAGS if f not in ("-fPIC", "-shared")]
    key = hashlib.sha256((B.source_hash(module) + " ".join(flags)).encode()).hexdigest()[:24]
    folder = os.path.join(tempfile.gettempdir(), f"gfa_isa_{os.getuid()}")
    os.makedirs(folder, exist_ok=True)
    path = os.path.join(folder, f"{module}_{key}.s")
    if not os.path.isfile(path):
        tmp = path + f".tmp{os.getpid()}"
        cmd = [B._hipcc()] + flags + ["-I", B.HERE, "-S", "--cuda-device-only",
                                      os.path.join(B.HERE, module + ".hip"), "-o", tmp]
        env = dict(os.environ)
        env.setdefault("HOME", tempfile.gettempdir())
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc -S failed on {module}.hip:\n{proc.stdout.decode()}")
        os.replace(tmp, path)
    with open(path) as f:
        return f.read()
