"""Build-time check of the compiled gfx950 code for one hazard of the step loops (csrc/ssd_chain_kernel.h, ssd_quad.hip).

Those loops read their B operands with `ds_read_b64_tr_b16` in inline assembly and wait for them in a later inline
assembly statement (`s_waitcnt lgkmcnt(n)`), so that several reads are in flight while matrix instructions run.  The
compiler takes the result registers of the first statement for complete.  Under register pressure, or to carry such a
value around a loop, it may copy them to other registers (`v_accvgpr_write`, `v_mov`) or reuse them between the two
statements -- the copy then holds whatever the register held before the data arrived, and results are silently wrong.
Nothing in the source can forbid that, so the generated code is checked: between a transposing read and the first
matrix instruction that takes its result registers as an operand, no other instruction may read or write them.

The chain kernel reads a step's x and weight operands the same way (`ds_read2st64_b32`, `ds_read_b128` inside an inline
assembly statement, waited for by the statement whose text ends in "; operands"): between such a read and that wait no
instruction may touch its result registers either.  Reads of those kinds that the compiler issues itself are its own
business and are not looked at.

check_text(asm) -> list of findings (empty = clean); check_file(path) the same for a file."""
import re

_REG = re.compile(r"^v\[(\d+):(\d+)\]$|^v(\d+)$")


def _regs(token):
    m = _REG.match(token)
    if not m:
        return set()
    if m.group(3) is not None:
        return {int(m.group(3))}
    return set(range(int(m.group(1)), int(m.group(2)) + 1))


def check_text(text, window=600):
    lines = text.split("\n")
    findings = []
    kernel = "?"
    for i, line in enumerate(lines):
        stripped = line.strip()
        if stripped.endswith(":") and not stripped.startswith(".") and not stripped.startswith(";"):
            kernel = stripped[:-1]
        if not stripped.startswith("ds_read_b64_tr_b16"):
            continue
        dst = _regs(re.split(r"[ ,]+", stripped)[1])
        for k in range(i + 1, min(i + window, len(lines))):
            t = lines[k].strip()
            if not t or t[0] in ";." or t.endswith(":"):
                continue
            parts = re.split(r"[ ,]+", t)
            op = parts[0]
            if op == "s_endpgm":
                break
            written = _regs(parts[1]) if len(parts) > 1 else set()
            read = set()
            for tok in parts[2:]:
                read |= _regs(tok)
            if op.startswith("buffer_store") or op.startswith("global_store") or op.startswith("ds_write"):
                read |= written          # stores read their first operand
                written = set()
            if op.startswith("v_mfma") and (read & dst):
                break                    # the consumer
            if op.startswith("ds_read_b64_tr_b16") and not (written & dst):
                continue
            if (read | written) & dst:
                findings.append({"kernel": kernel, "line": k + 1, "instruction": t, "loaded_at": i + 1,
                                 "registers": sorted((read | written) & dst)})
                break
    return findings


def check_operand_reads(text, window=400):
    """Inline-assembly x / weight reads: result registers untouched up to the "; operands" wait."""
    lines = text.split("\n")
    findings = []
    kernel = "?"
    in_asm = False
    for i, line in enumerate(lines):
        stripped = line.strip()
        if stripped.endswith(":") and not stripped.startswith(".") and not stripped.startswith(";"):
            kernel = stripped[:-1]
        if stripped.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if stripped.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not in_asm or not (stripped.startswith("ds_read2st64_b32") or stripped.startswith("ds_read_b128")):
            continue
        dst = _regs(re.split(r"[ ,]+", stripped)[1])
        done = False
        for k in range(i + 1, min(i + window, len(lines))):
            t = lines[k].strip()
            if "; operands" in t:
                done = True
                break
            if not t or t[0] in ";." or t.endswith(":"):
                continue
            parts = re.split(r"[ ,]+", t)
            touched = set()
            for tok in parts[1:]:
                touched |= _regs(tok)
            if touched & dst:
                findings.append({"kernel": kernel, "line": k + 1, "instruction": t, "loaded_at": i + 1,
                                 "registers": sorted(touched & dst)})
                done = True
                break
        if not done:
            findings.append({"kernel": kernel, "line": i + 1, "instruction": stripped, "loaded_at": i + 1,
                             "registers": sorted(dst), "note": "no wait for these operands in sight"})
    return findings


def check_file(path):
    with open(path) as f:
        text = f.read()
    return check_text(text) + check_operand_reads(text)
