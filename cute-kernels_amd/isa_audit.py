"""Checks the hand-counted waits of the streaming grouped-GEMM kernels against the compiler's assembly output.

Usage: python cute-kernels_amd/isa_audit.py [file.s]

The kernels of csrc/grouped_gemm_ragged.hip wait for their operand loads with `s_waitcnt vmcnt(N)` where N is a constant
that counts the vector-memory instructions a wavefront has issued after the loads it waits for (loads and stores complete
in issue order). The constants are derived in the source from the number of loads per K step, the number of stores an
epilogue issues and whether a prefetch, a bias load or a request for row_index entries follows a step's loads. This script
compiles the source to assembly (device code only; or reads a file made with `hipcc ... --cuda-device-only -S`) and checks,
for every instantiation of ragged_gemm_kernel, that the instruction stream has the shape those constants assume:

 * every wait that is followed by a barrier and the eight operand loads of a K step allows exactly the number of newer
   instructions of a step in the loop (prefetch, request) or of a tile's first step (the epilogue's stores, prefetch, bias);
 * between the two barriers of a loop body of two K steps a wavefront issues the eight loads and exactly those extras;
 * the cold start issues sixteen operand loads, as many stand-in stores as an epilogue issues stores, and waits for all but
   the eight loads of the second step and the stores;
 * the three-stage loop of groups of at most 64 rows issues five loads per step and waits for all but five;
 * no instantiation touches scratch memory, and none contains a loop over the distinct values of an operand that the
   hardware wants in scalar registers (what the compiler generates around a vector-memory instruction whose descriptor or
   scalar offset it cannot prove to be the same in every lane: each costs a dozen instructions and a branch per use).

The kernels that gather the rows of their first operand (forward form) read a row table between a step's barrier and its
loads, which spreads a step over several basic blocks in ways that differ from version to version of the loop: for them
only the loop bodies of two steps, the scratch memory and the loops over scalar operands are checked.
"""

import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(HERE, "csrc", "grouped_gemm_ragged.hip")
EPI_STORES = {0: 16, 1: 24, 2: 8, 3: 32}  # stores per wavefront and tile: plain, SwiGLU with h, SwiGLU, SwiGLU backward


def compile_to_assembly(path: str) -> None:
    from build import FLAGS, HIPCC  # the flags the library is built with

    cmd = [HIPCC] + FLAGS + ["--cuda-device-only", "-S", SOURCE, "-o", path]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(proc.stderr[-2000:])


def tokens(lines):
    """The vector-memory instructions, waits and barriers of a kernel in program order, and the number of loops over the
    distinct values of a scalar operand (readfirstlane, compare, s_and_saveexec, the instruction, s_xor exec, branch)."""
    cur, waterfalls = [], 0
    for k, line in enumerate(lines):
        s = line.strip()
        if s.startswith("s_cbranch_execnz") and any("s_xor_b64 exec, exec" in x for x in lines[max(0, k - 3):k]):
            waterfalls += 1
        if re.match(r"^\.LBB\d+_\d+:", line):
            cur.append(" ")
        elif s.startswith("s_barrier"):
            cur.append("|")
        elif s.startswith("s_waitcnt") and "vmcnt" in s:
            cur.append("w%s," % re.search(r"vmcnt\((\d+)\)", s).group(1))
        elif s.startswith("buffer_load_dwordx4") and " lds" in s:
            cur.append("O")  # sixteen bytes per lane into LDS: an operand load
        elif s.startswith("buffer_load_dword ") and " lds" in s:
            cur.append("p")  # four bytes per lane into LDS: prefetch, bias, row table, row_index request across a tile boundary
        elif s.startswith("buffer_load") or s.startswith("global_load"):
            cur.append("L")  # a load into registers
        elif s.startswith("buffer_store") or s.startswith("global_store"):
            cur.append("s")
        elif s.startswith("scratch_"):
            cur.append("X")
    return [b for b in "".join(cur).split(" ") if b], waterfalls


def audit(asm_path: str) -> int:
    lines = open(asm_path).read().split("\n")
    starts = [i for i, line in enumerate(lines) if re.match(r"^_ZN6fmahip4gemm6ragged18ragged_gemm_kernel.*:", line)]
    if not starts:
        raise RuntimeError("no ragged_gemm_kernel in " + asm_path)
    starts.append(len(lines))
    problems = 0
    for a, b in zip(starts[:-1], starts[1:]):
        name = lines[a].split(":")[0]
        m = re.search(r"ragged_gemm_kernelINS0_(\w+?)ELb(\d)ELb(\d)ELi(\d)ELb(\d)ELb(\d)ELb(\d)E", name)
        el, a_kc, b_kc, epi, vary_k, bias, gather = m.group(1), *[int(x) for x in m.groups()[1:]]
        body = lines[a:b]
        end = next((k for k, line in enumerate(body) if "s_endpgm" in line), len(body))
        blocks, waterfalls = tokens(body[:end])
        prefetch = 1 if a_kc == b_kc else 0
        request = 1 if (vary_k and gather) else 0
        stores = EPI_STORES[epi]
        wait_step, wait_first = prefetch + request, stores + prefetch + bias
        tag = f"{el} A_KC={a_kc} B_KC={b_kc} epilogue={epi} reduction_varies={vary_k} bias={bias} gather={gather}"
        found = {"step": 0, "first": 0, "body": 0, "cold": 0, "thin": 0}
        gathers_rows = bool(gather and not vary_k)

        def fail(what, block):
            nonlocal problems
            problems += 1
            print(f"PROBLEM {tag}: {what}: {block[:120]}")

        if waterfalls:
            fail(f"{waterfalls} loops over the distinct values of a scalar operand", "")
        for blk in blocks:
            if "X" in blk:
                fail("scratch access", blk)
            # waits in front of a barrier that the operand loads of a K step follow
            for w, loads in ([] if gathers_rows else re.findall(r"w(\d+),\|(O+)", blk)):
                n, count = int(w), len(loads)
                if count == 8:
                    if n == wait_step:
                        found["step"] += 1
                    elif n == wait_first:
                        found["first"] += 1
                    elif n == 8 + stores:
                        pass  # (the cold start's wait directly followed by the first step: not a shape the compiler produces)
                    else:
                        fail(f"a step waits for all but {n}, expected {wait_step} or {wait_first}", blk)
                elif count == 5:
                    if n == 5:
                        found["thin"] += 1
                    else:
                        fail(f"a three-stage step waits for all but {n}, expected 5", blk)
            # a loop body of two steps in one block: what is issued between its two barriers
            for between in re.findall(r"\|(O{8}[^|]*?)w\d+,\|O{8}", blk):
                issued = len(re.sub(r"w\d+,", "", between))
                if issued == 8 + wait_step:
                    found["body"] += 1
                else:
                    fail(f"{issued} instructions between the barriers of two steps, expected {8 + wait_step}", blk)
            # the cold start: sixteen operand loads (the gathered kinds mix loads of row_index entries in), the stand-in
            # stores, the wait
            cold = None if gathers_rows else re.search(r"((?:[OLp]|w\d+,)*O)(s+)w(\d+),\|", blk)
            if cold and cold.group(1).count("O") >= 16:
                found["cold"] += 1
                if cold.group(1).count("O") != 16 or len(cold.group(2)) != stores or int(cold.group(3)) != 8 + stores:
                    fail(f"cold start: {cold.group(1).count('O')} loads, {len(cold.group(2))} stores, wait {cold.group(3)}; "
                         f"expected 16, {stores}, {8 + stores}", blk)
        if gathers_rows:
            if found["body"] == 0:
                fail(f"expected shapes not found ({found})", "")
        else:
            if found["step"] == 0 or found["first"] == 0 or found["cold"] != 1:
                fail(f"expected shapes not found ({found})", "")
            if a_kc and found["thin"] == 0:
                fail("no three-stage loop found", "")
        print(f"ok  {tag}: steps {found['step']}, first steps {found['first']}, two-step bodies {found['body']}, "
              f"three-stage steps {found['thin']}")
    return problems


def main() -> int:
    if len(sys.argv) > 1:
        return audit(sys.argv[1])
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "grouped_gemm_ragged.s")
        sys.path.insert(0, HERE)
        compile_to_assembly(path)
        return audit(path)


if __name__ == "__main__":
    n = main()
    print("audit passed" if n == 0 else f"{n} problem(s)")
    sys.exit(0 if n == 0 else 1)
