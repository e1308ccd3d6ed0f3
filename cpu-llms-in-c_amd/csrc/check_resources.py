#!/usr/bin/env python3
"""Build step: reads the compiler's kernel-resource-usage remarks of one object file and fails the
build when a kernel has left the register, scratch or LDS budget that its launch shape relies on.

    check_resources.py <compiler log>

The log is the compiler's whole diagnostic output; what is not a resource remark (warnings, errors)
is passed through to stdout, the remarks themselves are only read.

Budgets (a kernel name is matched after demangling):
  * every q4_stream_kernel, q4_chain_kernel and q4_gemm_pipe_kernel instantiation: no scratch memory
    (a spill inside the streaming loop costs more than any occupancy it buys) and no spilled registers;
  * q4_stream_kernel<1, 1, 2, 16, *, false>: at most 64 vector registers - with sixteen waves a
    workgroup, two workgroups share a compute unit only up to 64 (one more halves the occupancy
    and the launch of the 27B q|k|v group takes a quarter longer);
  * q4_gemm_pipe_kernel: static LDS + the four 32 KiB activation stages it asks for at launch within
    the 160 KiB of a compute unit, and vector + accumulation registers within the 512 of a lane.
"""
import re
import subprocess
import sys

PIPE_DYNAMIC_LDS = 4 * 128 * 16 * 16
LDS_PER_CU = 160 * 1024


def kernels(text):
    for block in re.split(r"remark: Function Name: ", text)[1:]:
        name = block.split(" ", 1)[0]

        def field(label):
            found = re.search(re.escape(label) + r": (\d+)", block)
            return int(found.group(1)) if found else 0

        yield name, {"vgprs": field("VGPRs"), "agprs": field("AGPRs"),
                     "scratch": field("ScratchSize [bytes/lane]"), "vgpr_spill": field("VGPRs Spill"),
                     "sgpr_spill": field("SGPRs Spill"), "lds": field("LDS Size [bytes/block]")}


def split_log(text):
    """(remark lines, everything else): a remark is followed by the source line it points at and a
    caret line, and may be preceded by 'In file included from' lines."""
    remarks, others, held = [], [], []
    lines = text.splitlines()
    i = 0
    while i < len(lines):
        line = lines[i]
        if "[-Rpass-analysis=kernel-resource-usage]" in line:
            remarks.append(line)
            held = []
            i += 1
            while i < len(lines) and re.match(r"^\s*(\d+)?\s*\|", lines[i]):
                i += 1
            continue
        if line.startswith("In file included from") or "is not a recognized feature" in line:
            held.append(line)
        else:
            others.extend(h for h in held if "is not a recognized feature" not in h)
            held = []
            others.append(line)
        i += 1
    return "\n".join(remarks), [o for o in others if o.strip() and not re.match(r"^\d+ warnings? generated", o)]


def main():
    text, others = split_log(open(sys.argv[1]).read())
    for line in others:
        print(line)
    found = list(kernels(text))
    if not found:
        return 0  # a host-only object
    demangled = subprocess.run(["c++filt"], input="\n".join(name for name, _ in found), capture_output=True,
                               text=True, check=True).stdout.splitlines()
    problems = []
    for (mangled, use), name in zip(found, demangled):
        watched = re.search(r"(q4_stream_kernel|q4_chain_kernel|q4_gemm_pipe_kernel)<([^>]*)>", name)
        if not watched:
            continue
        kind, parameters = watched.group(1), [p.strip() for p in watched.group(2).split(",")]
        label = "%s<%s>" % (kind, ", ".join(parameters))
        if use["scratch"] or use["vgpr_spill"]:
            problems.append("%s: %d bytes of scratch per lane, %d spilled vector registers"
                            % (label, use["scratch"], use["vgpr_spill"]))
        if kind == "q4_stream_kernel" and parameters[:4] == ["1", "1", "2", "16"] and parameters[5:6] != ["true"] \
                and use["vgprs"] > 64:
            problems.append("%s: %d vector registers, the sixteen-wave launch needs at most 64" % (label, use["vgprs"]))
        if kind == "q4_gemm_pipe_kernel":
            if use["lds"] + PIPE_DYNAMIC_LDS > LDS_PER_CU:
                problems.append("%s: %d bytes of static LDS + %d at launch exceed %d"
                                % (label, use["lds"], PIPE_DYNAMIC_LDS, LDS_PER_CU))
            if use["vgprs"] + use["agprs"] > 512:
                problems.append("%s: %d + %d registers" % (label, use["vgprs"], use["agprs"]))
    for line in problems:
        print("check_resources: " + line, file=sys.stderr)
    return 1 if problems else 0


if __name__ == "__main__":
    sys.exit(main())
