"""Reads the assembly that the compiler makes of this package's kernels and measures, along every path through a
kernel, how many wait states lie between a matrix product and the first other instruction that touches the registers
of its result.

The hardware does not hold such an instruction back until the product has finished: the compiler has to put enough
instructions (or ``s_nop``) between the two.  It does so along straight code and across the branches it makes itself,
and it has been seen not to where an unrolled loop is left early (a ``break`` that depends on a run-time count right
behind the products of a row tile): the way out was a short cut of two wait states from the last product to the read
of its sums, and a tile with a single token read unfinished scores now and then.  Eight wait states are what the
compiler itself keeps for these 16 x 16 x 32 products wherever it counts.
"""

from __future__ import annotations

import collections
import re

_REGISTERS = re.compile(r"\b([av])\[(\d+):(\d+)\]|\b([av])(\d+)\b")


def registers(text: str) -> set[tuple[str, int]]:
    found: set[tuple[str, int]] = set()
    for match in _REGISTERS.finditer(text):
        if match.group(1):
            found.update((match.group(1), i) for i in range(int(match.group(2)), int(match.group(3)) + 1))
        else:
            found.add((match.group(4), int(match.group(5))))
    return found


def kernels_of(assembly: str) -> list[tuple[str, list[str]]]:
    """(name, instructions and labels) of every function in an assembly listing."""
    kernels: list[tuple[str, list[str]]] = []
    body: list[str] | None = None
    for line in assembly.split("\n"):
        start = re.match(r"^(_Z\w+):", line)
        if start:
            body = []
            kernels.append((start.group(1), body))
            continue
        if line.startswith(".Lfunc_end"):
            body = None
            continue
        if body is None:
            continue
        text = line.split(";")[0].strip()
        if text:
            body.append(text)
    return kernels


def short_paths(body: list[str], need: int) -> list[tuple[int, str, str]]:
    """(wait states, product, use) for every use of a product's result registers that some path reaches in fewer than
    ``need`` wait states.  A product that accumulates into the same registers may follow at once and ends the path."""
    label_at = {line[:-1]: index for index, line in enumerate(body) if line.endswith(":")}

    def successors(index: int) -> list[int]:
        words = body[index].split()
        op = words[0] if words else ""
        after = [index + 1] if index + 1 < len(body) else []
        if op == "s_endpgm":
            return []
        if op == "s_branch":
            return [label_at[words[-1]]] if words[-1] in label_at else []
        if op.startswith("s_cbranch"):
            return ([label_at[words[-1]]] if words[-1] in label_at else []) + after
        return after

    def wait_states(line: str) -> int:
        words = line.split()
        if not words or line.endswith(":"):
            return 0
        return int(words[1]) + 1 if words[0] == "s_nop" else 1

    found = []
    for index, line in enumerate(body):
        if not line.startswith(("v_mfma", "v_smfma")):
            continue
        result = registers(line.split(",")[0])
        nearest: dict[int, int] = {}
        queue = collections.deque((following, 0) for following in successors(index))
        while queue:
            at, distance = queue.popleft()
            if distance >= need or nearest.get(at, need) <= distance:
                continue
            nearest[at] = distance
            use = body[at]
            words = use.split()
            if words and not use.endswith(":") and len(words) > 1:
                touched = registers(use.split(None, 1)[1]) & result
                if touched:
                    if words[0].startswith("v_mfma"):
                        accumulates = registers(use.split(",")[0]) | registers(use.split(",")[-1])
                        if not touched <= accumulates:
                            found.append((distance, line, use))
                    else:
                        found.append((distance, line, use))
                    continue
            for following in successors(at):
                queue.append((following, distance + wait_states(use)))
    return found
