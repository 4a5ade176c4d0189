"""The LDS-DMA extend kernel counts its own memory waits (hipcc does not model the DMA).  Two compiler
behaviours would silently cost the two tiles of prefetch the ring exists for, without failing any
parity test: a `s_waitcnt vmcnt(0)` inside the tile loop (a fence, an alias wait in front of a
ds_read_tr intrinsic, a wait for loads the compiler believes pending) and scratch spills in the loop.
This test compiles the headline instantiation to assembly (hipcc cross-compiles without a GPU) and
checks the loop's text.  DESIGN.md section 4.3."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.fixture(scope="module")
def dma_kernel_asm(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("isa") / "extend_mfma.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fno-honor-nans", "-DSP_EXTEND_ONLY_HEADLINE",
           "--cuda-device-only", "-S", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "scratchpad_amd", "csrc"),
           os.path.join(ROOT, "scratchpad_amd", "csrc", "extend_mfma.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    text = open(out).read()
    # bf16, D 128, GK 4, 8 waves, 16-bit pool, PLAIN, DMA (, not persistent)
    m = re.search(r"^(_ZN2sp18extend_mfma_kernelINS_8bf16_tagELi128ELi4ELi8ELb0ELb1ELb1(?:ELb0)?EEEvNS_10ExtendArgsE):[^\n]*\n(.*?)^\.Lfunc_end",
                  text, re.S | re.M)
    assert m, "headline LDS-DMA instantiation not found"
    return m.group(2)


def test_tile_loop_keeps_its_dma_in_flight(dma_kernel_asm):
    lines = [l.strip() for l in dma_kernel_asm.splitlines()]
    barriers = [i for i, l in enumerate(lines) if l.startswith("s_barrier")]
    assert len(barriers) >= 6, "prologue barrier + one per unrolled tile step + the epilogue's"
    loop = lines[barriers[0] + 1:barriers[-2]]            # between the prologue's barrier and the last tile step's (the
                                                          # epilogue has its own barrier behind a full drain)
    assert sum(l.startswith("global_load_lds_dwordx4") for l in loop) >= 16, "4 DMA pieces per tile step"
    drained = [l for l in loop if re.match(r"s_waitcnt.*vmcnt\(0\)", l)]
    assert not drained, f"the tile loop drains the DMA ring: {drained[:3]}"
    counted = [l for l in loop if re.match(r"s_waitcnt vmcnt\(8\)", l)]
    assert len(counted) >= 4, "the hand-counted wait of every tile step survives"
    assert not any("scratch_" in l for l in loop[:len(loop) // 2]), "no spills in the unrolled main loop"
    assert "ds_read_b64_tr_b16" in dma_kernel_asm and "v_mfma_f32_32x32x16_bf16" in dma_kernel_asm


# ----------------------------------------------------------------------------------------------- extend_w64.hip
# The 4 x 64-row kernel keeps O^T and the Q fragments in accumulation registers that only its asm text names.  For the
# compiler to be UNABLE to use one of them (it parks values there as soon as architectural registers run short, and an
# AGPR in any asm constraint or clobber makes all of them allocatable) the source never mentions one to it and is built
# for a 256-register budget: hipcc then reserves every AGPR - and writes a kernel descriptor and a metadata note without
# any.  The build compiles this file in stages (scratchpad_amd/build.py:compile_w64) and tools/w64_asm.py rewrites the
# device ASSEMBLY so that the assembler itself derives a descriptor - and a note - with the 256 accumulation registers
# (round 5; before, the linked library was byte-patched and its note disagreed).  What the parity tests cannot see
# until it is too late: that guarantee lost (a constraint someone adds), a library linked from a plain `hipcc -c`,
# scratch in the tile loop (its wait drains the DMA ring), the generated bodies drifting away from their generator.
W64_FLAGS = ["-fno-honor-nans", "-fno-slp-vectorize", "-std=c++20", "-mllvm", "-amdgpu-atomic-optimizer-strategy=None"]
LIB = os.path.join(ROOT, "scratchpad_amd", "lib", "libscratchpad_hip.so")


def _w64_tool():
    import sys
    sys.path.insert(0, os.path.join(ROOT, "tools"))
    try:
        import w64_asm
    finally:
        sys.path.pop(0)
    return w64_asm


def test_w64_generated_bodies_are_the_generators_output():
    r = subprocess.run(["python3", os.path.join(ROOT, "tools", "gen_extend_w64.py"), "--check"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr


def test_w64_build_flags_are_the_tested_ones():
    from scratchpad_amd import build
    assert build.PER_FILE_FLAGS["extend_w64.hip"] == W64_FLAGS


def test_w64_rewrite_refuses_a_different_register_layout():
    """tools/w64_asm.py rewrite: another ACCUM_OFFSET (a toolchain that allocates this source differently), or a
    compiler that uses accumulation registers itself, stops the build; kernels other than the w64 ones are untouched."""
    w = _w64_tool()

    def asm(name, nfv, accum, agpr=0):
        return (f"\t.amdhsa_kernel {name}\n\t\t.amdhsa_next_free_vgpr {nfv}\n\t\t.amdhsa_accum_offset {accum}\n"
                f"\t.end_amdhsa_kernel\n"), (f"  - .agpr_count:     {agpr}\n    .args:\n      - .name:           a\n"
                                              f"    .name:           {name}\n    .vgpr_count:     {nfv}\n")
    names = [f"_ZN2sp{len(k)}{k}INS_{t}EEEvNS_10ExtendArgsE" for k in w.KERNELS for t in ("8bf16_tag", "7f16_tag")]
    other = "_ZN2sp18extend_mfma_kernelIfEEvv"

    def text(accums):
        ks, ms = zip(*[asm(n, a - 1, a) for n, a in zip(names, accums)] + [asm(other, 90, 92, 4)])
        return "".join(ks) + "\t.amdgpu_metadata\n---\namdhsa.kernels:\n" + "".join(ms) + "...\n\t.end_amdgpu_metadata\n"
    good = [w.EXPECTED[w.kernel_of(n)] for n in names]
    out = w.rewrite(text(good))
    for n, a in zip(names, good):
        assert re.search(rf"\.amdhsa_kernel {n}\n\t\t\.amdhsa_next_free_vgpr {a + 256}\n", out)
        assert re.search(rf"- \.agpr_count:\s+256\n(?:(?!- \.agpr_count).)*?\n    \.name:\s+{n}\n\s+\.vgpr_count:\s+{a + 256}\n", out, re.S)
    assert f".amdhsa_kernel {other}\n\t\t.amdhsa_next_free_vgpr 90\n" in out and "- .agpr_count:     4\n" in out
    with pytest.raises(SystemExit, match="ACCUM_OFFSET"):
        w.rewrite(text([good[0] - 4] + good[1:]))
    with pytest.raises(SystemExit, match="allocates accumulation registers"):
        w.rewrite(text(good).replace(f".amdhsa_next_free_vgpr {good[0] - 1}\n", f".amdhsa_next_free_vgpr {good[0] + 8}\n", 1))


@pytest.fixture(scope="module")
def w64_asm(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("isa") / "extend_w64.s"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3"] + W64_FLAGS + [
        "--cuda-device-only", "-S", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "scratchpad_amd", "csrc"),
        os.path.join(ROOT, "scratchpad_amd", "csrc", "extend_w64.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    return open(out).read()


@pytest.mark.parametrize("tag", ["8bf16_tag", "7f16_tag"])
def test_w64_registers_belong_to_whom_they_should(w64_asm, tag):
    name = f"_ZN2sp17extend_w64_kernelINS_{tag}EEEvNS_10ExtendArgsE"
    m = re.search(rf"^{name}:[^\n]*\n(.*?)^\.Lfunc_end", w64_asm, re.S | re.M)
    assert m, "kernel not found"
    body = m.group(1)
    meta = re.search(rf"\.name:\s+{name}\n(.*?)\.wavefront_size", w64_asm, re.S)
    assert meta
    fields = dict(re.findall(r"\.(\w+):\s+(\d+)", meta.group(1)))
    agpr = re.search(rf"\.agpr_count:\s+(\d+)(?:(?!\.agpr_count).)*?\.name:\s+{name}\n", w64_asm, re.S)
    assert agpr and int(agpr.group(1)) == 0, "the compiler believes the kernel uses no accumulation register: all of them are reserved"
    assert int(fields["private_segment_fixed_size"]) == 0 and int(fields["vgpr_spill_count"]) == 0
    assert int(fields["vgpr_count"]) <= 256 - 8, "architectural registers: a margin below the 256 the build allows"
    assert "scratch_" not in body
    inside, mine, used = False, [], set()
    for line in body.splitlines():
        if "ASMSTART" in line:
            inside = True
        elif "ASMEND" in line:
            inside = False
        elif not inside and re.search(r"[ ,]a(\[|\d)", line.split(";")[0]):
            mine.append(line.strip())
        elif inside:
            for lo, hi in re.findall(r"\ba\[(\d+):(\d+)\]", line):
                used.update((int(lo), int(hi)))
            used.update(int(x) for x in re.findall(r"\ba(\d+)\b", line))
    assert not mine, f"compiler-made instructions touch accumulation registers: {mine[:4]}"
    assert max(used) == 191, "O^T a[0:127] + Q a[128:191]"
    lines = [l.strip() for l in body.splitlines()]
    bars = [i for i, l in enumerate(lines) if l == "s_barrier"]
    assert len(bars) >= 8
    # the pipelined bodies: the stretches between two barriers that issue a tile's 8 pieces
    bodies = [lines[bars[b]:bars[b + 1]] for b in range(len(bars) - 1)]
    bodies = [it for it in bodies if sum(l.startswith("global_load_lds") for l in it) == 8]
    assert len(bodies) >= 6, "four unrolled bodies, the loop's tail, minus the first one (its pieces precede the way in's barrier)"
    hot = [l for it in bodies for l in it]
    # an iteration's pieces go out in its first gaps; a full drain AHEAD of them only meets operations issued most of an
    # iteration ago (the compiler's wait for the indices), one behind them would wait for the pieces themselves
    # (a stretch runs from one body's barrier - gap 57 - to the next one's: 64 MFMAs between two bodies of the loop)
    assert sum(1 for it in bodies if sum(l.startswith("v_mfma_f32_32x32x16") for l in it) == 64) >= 4
    for it in bodies:
        first = next(i for i, l in enumerate(it) if l.startswith("global_load_lds"))
        assert not [l for l in it[first:] if re.match(r"s_waitcnt.*vmcnt\(0\)", l)], "the body drains its own DMA pieces"
        assert [l for l in it if re.match(r"s_waitcnt vmcnt\(16\)", l)], "the counted wait ahead of the barrier"
    assert not any(l.startswith("flat_load") for l in hot), "index loads must be global (a flat load counts in lgkmcnt)"
    assert not any(l.startswith("v_pk_") for l in hot), "packed f32 vector instructions beside the MFMAs"


@pytest.mark.parametrize("tag", ["8bf16_tag", "7f16_tag"])
def test_w64_persistent_form_keeps_to_its_registers(w64_asm, tag):
    """The persistent form of the kernel (extend_w64p_kernel): the same ownership rules, more accumulation registers in
    its asm text - the next item's kv slots in a[192:203], the second half of its Q rows in a[204:235] - and not one
    spilled value (a reload is a s_waitcnt vmcnt(0): a drained DMA ring in the middle of an item)."""
    name = f"_ZN2sp18extend_w64p_kernelINS_{tag}EEEvNS_10ExtendArgsE"
    m = re.search(rf"^{name}:[^\n]*\n(.*?)^\.Lfunc_end", w64_asm, re.S | re.M)
    assert m, "kernel not found"
    body = m.group(1)
    meta = re.search(rf"\.name:\s+{name}\n(.*?)\.wavefront_size", w64_asm, re.S)
    assert meta
    fields = dict(re.findall(r"\.(\w+):\s+(\d+)", meta.group(1)))
    agpr = re.search(rf"\.agpr_count:\s+(\d+)(?:(?!\.agpr_count).)*?\.name:\s+{name}\n", w64_asm, re.S)
    assert agpr and int(agpr.group(1)) == 0, "the compiler believes the kernel uses no accumulation register: all of them are reserved"
    assert int(fields["private_segment_fixed_size"]) == 0 and int(fields["vgpr_spill_count"]) == 0
    assert int(fields["vgpr_count"]) <= 256
    assert "scratch_" not in body
    inside, mine, used = False, [], set()
    for line in body.splitlines():
        if "ASMSTART" in line:
            inside = True
        elif "ASMEND" in line:
            inside = False
        elif not inside and re.search(r"[ ,]a(\[|\d)", line.split(";")[0]):
            mine.append(line.strip())
        elif inside:
            for lo, hi in re.findall(r"\ba\[(\d+):(\d+)\]", line):
                used.update((int(lo), int(hi)))
            used.update(int(x) for x in re.findall(r"\ba(\d+)\b", line))
    assert not mine, f"compiler-made instructions touch accumulation registers: {mine[:4]}"
    assert max(used) == 235, "O^T a[0:127], Q a[128:191], next kv slots a[192:203], next Q rows a[204:235]"
    # the ticket draw stays an atomic whose value is waited for where it is read (the atomic optimizer's form waits -
    # a full round trip - right behind it)
    lines = [l.strip() for l in body.splitlines()]
    draws = [i for i, l in enumerate(lines) if l.startswith("global_atomic_add") and "sc0" in l]
    waited = []
    for i in draws:
        nxt = [l for l in lines[i + 1:i + 8] if l and not l.startswith((";", "."))]
        waited.append(any(re.match(r"s_waitcnt.*vmcnt\(0\)", l) for l in nxt[:3]))
    # (the two completion counts at the kernel's ends are read at once; the draws inside the item loop are not)
    assert len(draws) >= 3 and waited.count(False) >= 2, "the ticket is waited for on the spot"
