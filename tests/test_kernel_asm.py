"""Static checks on the compiler's output for the hand-scheduled m > 16 kernel.

Its MFMAs and direct-to-LDS loads are inline asm, so the compiler's hazard recogniser does not see them; the
rules it would have enforced are checked here on the generated gfx950 assembly of the shipped source
(`hipcc -S --cuda-device-only`, about a minute, no GPU):

* no MFMA reads a VGPR/AGPR that a VALU instruction wrote fewer than two wait states earlier;
* every direct-to-LDS load in scalar-base form got SGPRs for its base and every M0 write an SGPR source
  (an "s" asm operand that the compiler could not prove uniform silently becomes a VGPR);
* the MFMA loops of the m > 16 kernels move no accumulator (no v_accvgpr_* inside them) and spill nothing.
"""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "fp6-marlin_amd", "csrc", "fp6m_gemm.hip")
HIPCC = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")


@pytest.fixture(scope="module")
def asm(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm") / "fp6m_gemm.s"
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                           "-packed-fp32-ops", f"-I{ROOT}/include", f"-I{ROOT}/fp6-marlin_amd/csrc", "-S",
                           "--cuda-device-only", "-o", str(out), SRC], stderr=subprocess.DEVNULL)
    return out.read_text()


def kernels(asm):
    for m in re.finditer(r"^(_ZN4fp6m\w+):", asm, re.M):
        if f".type\t{m.group(1)},@function" not in asm:                 # a data symbol (the static scratch array)
            continue
        body = asm[m.start():asm.index(".Lfunc_end", m.start())]
        ins = [l.strip() for l in body.split("\n") if l.startswith("\t") and l.strip() and not l.strip().startswith((".", ";"))]
        yield m.group(1), ins


def regs(tok):
    tok = tok.strip().rstrip(",")
    m = re.match(r"^([va])\[(\d+):(\d+)\]$", tok)
    if m:
        return {(m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"^([va])(\d+)$", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def test_no_valu_write_right_before_mfma_read(asm):
    checked = 0
    for name, ins in kernels(asm):
        for n, l in enumerate(ins):
            if not l.startswith("v_mfma"):
                continue
            checked += 1
            src = set().union(*[regs(o) for o in l.split(None, 1)[1].split(",")[1:4]])
            waited, k = 0, n - 1
            while k >= 0 and waited < 2:
                p = ins[k]
                if p.startswith("s_nop"):
                    waited += int(p.split()[1]) + 1
                else:
                    if p.startswith("v_") and not p.startswith("v_mfma"):
                        dst = regs(p.split(None, 1)[1].split(",")[0])
                        assert not (dst & src), f"{name}: `{p}` feeds `{l}` after {waited} wait states"
                    waited += 1
                k -= 1
    assert checked > 500


def test_scalar_operands_of_asm_loads(asm):
    assert not re.findall(r"global_load_lds_dwordx?4? v\d+, v[\[\d]", asm), "direct-to-LDS load with a vector base"
    assert not re.findall(r"s_mov_b32 m0, v\d", asm), "M0 written from a VGPR"
    assert not re.findall(r"global_load_dwordx2 v\[\d+:\d+\], v\d+, v[\[\d]", asm), "2-bit plane load with a vector base"
    assert len(re.findall(r"global_load_lds_dwordx4 v\d+, s\[", asm)) > 20


def test_mfma_loops_keep_accumulators_in_place(asm):
    seen = 0
    for name, ins in kernels(asm):
        if "gemm_mb_kernel" not in name:
            continue
        seen += 1
        meta = asm[asm.index(".name:           " + name) - 400:asm.index(".name:           " + name) + 800]
        # Between two MFMAs of one loop (fewer than 100 other instructions apart; what separates the FP6 loop from the
        # INT4 loop of the same kernel is longer: with the accumulators in the accumulation registers the deferred
        # FP6 re-bias reads and writes every one of them there) nothing may touch an accumulation register.
        mfmas = [n for n, l in enumerate(ins) if l.startswith("v_mfma")]
        moved = [l for a, b in zip(mfmas, mfmas[1:]) if b - a < 100 for l in ins[a:b] if l.startswith("v_accvgpr")]
        if "gemm_mb_kernelILb1ELi8E" in name or "gemm_mb_kernelILb0ELi8E" in name:
            # eight blocks: with all 256 accumulation registers taken the allocator permutes some accumulators through
            # ordinary registers at the back edge of its two loops (four k steps = 256 MFMAs per trip): bounded, not none
            assert len(moved) <= 300, f"{name}: {len(moved)} accumulator copies between MFMAs"
            continue
        assert not moved, f"{name}: accumulator copies between MFMAs: {moved[:4]}"
    # (group scales or not) x ((MB 2, MB 4, MB 4 with paired A fetches) x (4, 8 k slices) + MB 2 paired with 8 slices +
    # MB 8), a second build without the optional paths of those that the dispatcher picks by itself (6 x 2 less
    # one that would spill), and a third, with two classes of INT4 tiles, of two of those (2 x 2 less one that would spill)
    assert seen == 30
    assert not re.findall(r"\.vgpr_spill_count:\s+[1-9]", asm), "a kernel spills VGPRs"
    # nothing may live in private memory either: a pointer that the compiler keeps on the stack costs the decode loop a
    # scratch load and a full `s_waitcnt vmcnt(0)` per step (seen once with pointers advanced under uniform branches)
    assert not re.findall(r"\.private_segment_fixed_size:\s+[1-9]", asm), "a kernel uses scratch memory"
    assert "scratch_load" not in asm and "scratch_store" not in asm


def test_kernel_arguments_are_loaded_in_one_batch(asm):
    """Scalar loads of kernel arguments between the top of a GEMM kernel and its first MFMA would each add a dependent
    round trip before the first weight load (measured: 0.4 us per launch when the slice tables were read by computed
    index).  All of them must sit in the first few instructions, behind a single wait.  The decode kernel fetches its
    argument block itself: four loads, one wait, and no other argument load anywhere."""
    seen = 0
    for name, ins in kernels(asm):
        if not any(k in name for k in ("gemm_m16_kernel", "gemm_sk_kernel", "gemm_mb_kernel")):
            continue
        seen += 1
        if "gemm_sk_kernel" in name:
            loads = [n for n, l in enumerate(ins) if l.startswith("s_load") and "s[0:1]" in l]
            assert loads == [0, 1, 2, 3] and ins[4].startswith("s_waitcnt lgkmcnt(0)"), f"{name}: {ins[:6]}"
            continue
        first_mfma = next(n for n, l in enumerate(ins) if l.startswith("v_mfma"))
        late = [(n, l) for n, l in enumerate(ins[:first_mfma]) if l.startswith("s_load") and n > 16]
        # the code of the epilogue may be laid out ahead of the loops: its loads (fused-epilogue pointers) do not count
        late = [(n, l) for n, l in late if not re.search(r"0x(c8|d0|d8)$", l)]
        assert not late, f"{name}: kernel-argument loads after the prologue: {late[:4]}"
    assert seen == 72            # (the m <= 16 kernel's builds with the partial tiles exchanged inside one XCD are 8 of them)
