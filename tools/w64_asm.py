#!/usr/bin/env python3
"""Give the extend_w64 kernels the accumulation registers their assembly text uses - AT ASSEMBLY LEVEL.

extend_w64.hip keeps O^T and the Q fragments in a[0:191] (the persistent form: a[0:235]), named only inside
`asm volatile` text.  For the compiler to be UNABLE to put anything of its own there (it does, as soon as architectural
registers run short, and an AGPR named in any asm constraint or clobber makes all of them allocatable), the source never
mentions an accumulation register to it and is built for a 256-register budget (__launch_bounds__(256, 2)): hipcc then
reserves every AGPR, and the kernel descriptor and metadata it writes allocate none.

Until round 4 a script raised GRANULATED_WORKITEM_VGPR_COUNT in the descriptors of the LINKED library (byte surgery; the
.amdgpu_metadata note kept saying agpr_count 0).  Now the build (scratchpad_amd/build.py) compiles this one file in
stages - device assembly (`hipcc --cuda-device-only -S`), THIS rewrite, `clang -x assembler`, lld, the offload bundle,
the host object with `-fcuda-include-gpubinary` - and the rewrite edits the two places the compiler states the
allocation, for the kernels named in KERNELS only:

  .amdhsa_next_free_vgpr  N   ->  ACCUM_OFFSET + 256     (gfx90a+: the unified total = accum offset + AGPRs; the
                                                           assembler derives the descriptor's granule count from it
                                                           and validates it against the register file)
  .amdgpu_metadata:  .agpr_count 0 -> 256,  .vgpr_count N -> ACCUM_OFFSET + 256

so descriptor and note agree and nothing is patched after linking.  The kernels' text addresses a[i] on the assumption
that the compiler keeps its own values in v[0:ACCUM_OFFSET): a toolchain that lays the register file out differently
(another ACCUM_OFFSET for the same source) fails the build here (EXPECTED), to be looked at by a person.

  python tools/w64_asm.py rewrite IN.s OUT.s      # the build step
"""
import re
import sys

W64_AGPRS = 256     # a[0:191] O^T and Q; a[192:235]: the persistent form (the next item's kv slots and half of its Q rows)
KERNELS = ("extend_w64_kernel", "extend_w64p_kernel")
# kernel -> ACCUM_OFFSET with hipcc of ROCm 7.2.0 (build.py records the compiler version next to the library)
EXPECTED = {"extend_w64_kernel": 228, "extend_w64p_kernel": 248}


def kernel_of(symbol: str):
    for k in KERNELS:
        if "2sp%d%sI" % (len(k), k) in symbol:
            return k
    return None


def rewrite(text: str) -> str:
    out, seen = [], {}
    lines = text.split("\n")
    i = 0
    # ---- the .amdhsa_kernel blocks
    cur = None
    block_start = None
    for idx, line in enumerate(lines):
        m = re.match(r"\s*\.amdhsa_kernel\s+(\S+)", line)
        if m:
            cur, block_start = (m.group(1) if kernel_of(m.group(1)) else None), idx
        elif re.match(r"\s*\.end_amdhsa_kernel", line):
            if cur:
                blk = range(block_start, idx)
                acc = [j for j in blk if re.match(r"\s*\.amdhsa_accum_offset\s+\d+", lines[j])]
                nfv = [j for j in blk if re.match(r"\s*\.amdhsa_next_free_vgpr\s+\d+", lines[j])]
                assert len(acc) == 1 and len(nfv) == 1, f"{cur}: descriptor directives not found"
                accum = int(lines[acc[0]].split()[-1])
                have = int(lines[nfv[0]].split()[-1])
                want = EXPECTED[kernel_of(cur)]
                if accum != want:
                    raise SystemExit(f"{cur}: ACCUM_OFFSET {accum}, expected {want}: the compiler lays this kernel's registers "
                                     "out differently from the toolchain extend_w64.hip was written against - inspect before use")
                if have > accum:
                    raise SystemExit(f"{cur}: the compiler itself allocates accumulation registers (next_free_vgpr {have} > "
                                     f"accum_offset {accum}): the asm text's a[0:{W64_AGPRS - 1}] would collide with them")
                lines[nfv[0]] = re.sub(r"\d+\s*$", str(accum + W64_AGPRS), lines[nfv[0]])
                seen[cur] = accum
            cur = None
    # ---- the metadata note (YAML between .amdgpu_metadata and .end_amdgpu_metadata): one entry per kernel, "  - " opens it
    try:
        a = next(j for j, l in enumerate(lines) if l.strip() == ".amdgpu_metadata")
        b = next(j for j, l in enumerate(lines) if l.strip() == ".end_amdgpu_metadata")
    except StopIteration:
        raise SystemExit("no .amdgpu_metadata block in the assembly")
    starts = [j for j in range(a, b) if lines[j].startswith("  - .") and not lines[j].startswith("      ")]
    starts = [j for j in starts if re.match(r"  - \.\w+:", lines[j])]
    noted = set()
    for n, s in enumerate(starts):
        e = starts[n + 1] if n + 1 < len(starts) else b
        name = next((re.match(r"\s+\.name:\s+(\S+)", lines[j]).group(1) for j in range(s, e)
                     if re.match(r"\s+\.name:\s+\S+", lines[j]) and not lines[j].startswith("      ")), None)
        if name not in seen:
            continue
        for j in range(s, e):
            if re.match(r"\s+(- )?\.agpr_count:\s+\d+", lines[j]) and not lines[j].startswith("      "):
                lines[j] = re.sub(r"\d+\s*$", str(W64_AGPRS), lines[j])
            elif re.match(r"\s+(- )?\.vgpr_count:\s+\d+", lines[j]) and not lines[j].startswith("      "):
                lines[j] = re.sub(r"\d+\s*$", str(seen[name] + W64_AGPRS), lines[j])
        noted.add(name)
    if len(seen) != 2 * len(KERNELS) or noted != set(seen):
        raise SystemExit(f"expected {2 * len(KERNELS)} w64 kernels with descriptor and note, found descriptors {sorted(seen)}, notes {sorted(noted)}")
    return "\n".join(lines)


def main():
    if len(sys.argv) >= 4 and sys.argv[1] == "rewrite":
        open(sys.argv[3], "w").write(rewrite(open(sys.argv[2]).read()))
    else:
        print(__doc__)
        sys.exit(2)


if __name__ == "__main__":
    main()
