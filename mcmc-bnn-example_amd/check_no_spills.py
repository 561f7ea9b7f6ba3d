#!/usr/bin/env python3
"""Build check: the kernels whose tile loads are issued from inline assembly must not spill.

Such a load lands in its register long after the compiler believes the register written; if the
register is spilled to scratch or re-used while the load is in flight, the kernel computes with, or
addresses memory through, corrupted values.  Reads the -Rpass-analysis=kernel-resource-usage remarks of
a compilation and fails if one of those kernels has VGPR spills or uses scratch memory, or if the
file holds none of them.  (Every other inline-assembly load of the library waits for its result inside
the same assembly statement, so the kernels that use only those may spill freely.)"""
import re
import sys

ASM_LOAD_KERNELS = ("MfmaLayerILi22ELi40ELi2EEE", "MfmaHybridLayer", "hmc_kernel_wide")


def main(path):
    text = open(path, errors="replace").read()
    blocks = re.split(r"remark: Function Name: ", text)[1:]
    checked, bad = 0, []
    for b in blocks:
        name = b.split()[0]
        if not any(k in name for k in ASM_LOAD_KERNELS):
            continue
        checked += 1
        spill = int(re.search(r"VGPRs Spill: (\d+)", b).group(1))
        scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b).group(1))
        if spill or scratch:
            bad.append("%s: %d VGPRs spilled, %d bytes of scratch per lane" % (name, spill, scratch))
    for line in bad:
        print("check_no_spills: " + line, file=sys.stderr)
    if bad:
        return 1
    if checked == 0:
        print("check_no_spills: no kernel in %s matches %s: the check would be vacuous" % (
            path, ", ".join(ASM_LOAD_KERNELS)), file=sys.stderr)
        return 1
    print("check_no_spills: %d kernel(s) with assembly-issued loads in %s, none spills" % (checked, path))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1]))
