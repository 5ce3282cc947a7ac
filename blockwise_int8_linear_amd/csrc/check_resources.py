"""Reads hipcc's -Rpass-analysis=kernel-resource-usage remarks of one translation unit (a file of hipcc's stderr), passes every
other line of it on to stderr, and fails if a kernel spills registers beyond what is known and accepted.

The GEMM kernels count their own loads in flight (`s_waitcnt vmcnt(n)` with hand-computed n).  Spill code adds loads and
stores of its own to that queue: the waits stay correct (memory instructions of a wave complete in order, so an extra one only
makes a wait stricter), but a spill inside a K loop costs far more than the instructions it saves -- the 64-column form of
gemm_panel at block 64 spilled 20 registers and took 46 us where 29 were to be had -- so a build that starts to spill says so.
usage: check_resources.py REMARKS_FILE"""
import re
import subprocess
import sys

# kernel name prefix (demangled, without the namespace) -> spilled VGPRs that are known: outside the K loops, measured harmless
ACCEPTED = {"gemm_wide32<32,": 8, "gemm_wide<64, 0, 8, false>": 4, "gemm_wide<128, 0, 8, false>": 4, "gemm_tile<256, 128, 4, 2, 3, 64, 0, true, false>": 2}


def main(path):
    name, bad = None, []
    for line in open(path, errors="replace"):
        if "[-Rpass-analysis=kernel-resource-usage]" not in line:
            sys.stderr.write(line)
            continue
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"VGPRs Spill: (\d+)", line)
        if m and int(m.group(1)) > 0:
            bad.append((name, int(m.group(1))))
    failed = False
    for mangled, n in bad:
        plain = subprocess.run(["c++filt", mangled], capture_output=True, text=True).stdout.strip()
        plain = plain.replace("(anonymous namespace)::", "").replace("void ", "")
        allowed = max([v for k, v in ACCEPTED.items() if plain.startswith(k)] or [0])
        if n > allowed:
            sys.stderr.write(f"check_resources: {plain} spills {n} VGPRs (accepted: {allowed})\n")
            failed = True
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1]))
