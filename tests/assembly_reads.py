"""A check on the compiler's assembly of a HIP source whose LDS reads are written as inline
assembly with waits of their own (``pagedserve_amd/csrc/attention_prefill.hip``).

The compiler does not know that a register which such a read fills is still on its way: it
may copy or overwrite it as soon as the statement has been issued.  The source keeps every
such register on one straight path, read, wait, use, so that nothing touches it in between.
This module verifies that on the assembly: a forward data-flow over the basic blocks of every
kernel, in which a register is *pending* from the read that names it as destination until a
``s_waitcnt lgkmcnt(n)`` covers that read.  Where paths meet, a register is pending if it is on
any of them.  ``lgkmcnt(0)`` clears everything; ``lgkmcnt(n)`` clears everything but the last n
reads where the block itself issued at least n (reads return in the order of issue), and,
conservatively, nothing otherwise.  Any other instruction that names a pending register is
reported.  Only reads between the assembler's ``#ASMSTART`` / ``#ASMEND`` marks are tracked: the
compiler waits for its own.
"""

import re

_REG_RANGE = re.compile(r"v\[(\d+):(\d+)\]")
_REG_ONE = re.compile(r"\bv(\d+)\b")
_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_READ = re.compile(r"ds_read\w*\s+(v\[(\d+):(\d+)\]|v(\d+))")
_WAIT = re.compile(r"s_waitcnt.*lgkmcnt\((\d+)\)")


def _registers(text):
    used = set()
    for first, last in _REG_RANGE.findall(text):
        used |= set(range(int(first), int(last) + 1))
    for number in _REG_ONE.findall(text):
        used.add(int(number))
    return used


def _blocks_of(body):
    """(basic blocks as lists of instructions with ASM marks, successors of each)."""
    blocks, labels, current = [], {}, []
    for line in body.split(".Lfunc_end")[0].splitlines()[1:]:
        if ";;#ASMSTART" in line:
            current.append("#ASMSTART")
            continue
        if ";;#ASMEND" in line:
            current.append("#ASMEND")
            continue
        code = line.split(";")[0].strip()
        if not code:
            continue
        label = _LABEL.match(code)
        if label:
            if current:
                blocks.append(current)
                current = []
            labels[label.group(1)] = len(blocks)
            continue
        if code.startswith("."):
            continue
        current.append(code)
        if code.startswith(("s_branch", "s_cbranch", "s_endpgm")):
            blocks.append(current)
            current = []
    if current:
        blocks.append(current)
    successors = []
    for index, block in enumerate(blocks):
        real = [code for code in block if not code.startswith("#")]
        last = real[-1] if real else ""
        out = []
        if last.startswith("s_branch"):
            out.append(labels[last.split()[1]])
        elif last.startswith("s_cbranch"):
            out.append(labels[last.split()[1]])
            if index + 1 < len(blocks):
                out.append(index + 1)
        elif not last.startswith("s_endpgm") and index + 1 < len(blocks):
            out.append(index + 1)
        successors.append(out)
    return blocks, successors


def _run(block, pending_in, report):
    pending = set(pending_in)
    issued = []          # this block's reads in order: the registers each one fills, if tracked
    problems = []
    in_asm = False
    for code in block:
        if code == "#ASMSTART":
            in_asm = True
            continue
        if code == "#ASMEND":
            in_asm = False
            continue
        read = _READ.match(code)
        if read:
            if read.group(2):
                target = set(range(int(read.group(2)), int(read.group(3)) + 1))
            else:
                target = {int(read.group(4))}
            address = _registers(code.split(",", 1)[1]) if "," in code else set()
            if report and address & pending:
                problems.append((code, sorted(address & pending)))
            issued.append(target if in_asm else set())
            if in_asm:
                pending |= target
            continue
        wait = _WAIT.match(code)
        if wait:
            left = int(wait.group(1))
            if left == 0:
                pending, issued = set(), []
            elif len(issued) >= left:
                issued = issued[len(issued) - left:]
                pending = set().union(*issued)
            continue
        if code.startswith("s_"):
            continue
        touched = _registers(code) & pending
        if report and touched:
            problems.append((code, sorted(touched)))
    return pending, problems


def registers_touched_in_flight(assembly: str, kernel_prefix: str):
    """{kernel name: [(instruction, registers)]} for every kernel whose mangled name starts
    with ``kernel_prefix``; an empty list means that the kernel is clean."""
    found = {}
    for body in re.split(r"\n(?=" + re.escape(kernel_prefix) + r"\w+:)", assembly)[1:]:
        name = body.split(":", 1)[0]
        blocks, successors = _blocks_of(body)
        state = [set() for _ in blocks]
        work = list(range(len(blocks)))
        while work:
            index = work.pop(0)
            out, _ = _run(blocks[index], state[index], False)
            for follower in successors[index]:
                if not out <= state[follower]:
                    state[follower] |= out
                    if follower not in work:
                        work.append(follower)
        problems = []
        for index, block in enumerate(blocks):
            problems += _run(block, state[index], True)[1]
        found[name] = problems
    return found
