"""Code-generation checks of the MFMA GEMM kernels (no GPU needed: hipcc
cross-compiles).  The main-loop MFMAs of the one-wave-per-SIMD kernel are inline
assembly, so the compiler knows neither their latency nor that they are MFMAs;
these tests pin the properties the kernel's correctness argument relies on."""

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm") / "gemm_bf16.s"
    src = os.path.join(ROOT, "axonn_amd", "csrc", "gemm_bf16.hip")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.dirname(src),
           "--cuda-device-only", "-S", src, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=900)
    text = out.read_text()
    kernels = {}
    for m in re.finditer(r"^(_ZN3axn\S*gemm_(?:(?:bf16|f16)_(?:solo|rest|swiglu)|backward)_kernel\S*):", text, re.M):
        end = text.index(".end_amdhsa_kernel", m.end())
        kernels[m.group(1)] = text[m.end():end]
    # 7 layout/epilogue/output variants x 3 tile shapes (256 x 256, 128 x 128, 256 x 128) x 2 element
    # types (and the two-term input gradient as an eighth variant), and the gate/up forward of
    # each type
    assert len(kernels) >= 50, sorted(kernels)
    return kernels


def _instructions(body):
    return [ln.split(";")[0].strip() for ln in body.split("\n") if ln.split(";")[0].strip()]


def test_solo_kernels_do_not_spill(gemm_asm):
    for name, body in gemm_asm.items():
        assert re.search(r"\.amdhsa_private_segment_fixed_size 0\b", body), name
        assert "scratch_" not in body, name


def test_accumulators_stay_in_their_registers_until_the_last_mfma_has_retired(gemm_asm):
    """An accumulator copied out of its AGPRs right behind the MFMA that writes it is
    read before the result has left the pipeline.  So: every v_accvgpr_read follows
    the textually preceding MFMA by at least 32 idle cycles (two s_nop 15), and no
    basic block moves AGPRs around (v_accvgpr_mov: the zero-initialisation) behind
    an MFMA of its own."""
    for name, body in gemm_asm.items():
        ins = _instructions(body)
        nops, reads, mfma_in_block = 2, 0, False
        for s in ins:
            if s.startswith(".LBB"):
                mfma_in_block = False
            elif s.startswith("v_mfma"):
                nops, mfma_in_block = 0, True
            elif s == "s_nop 15":
                nops += 1
            elif s.startswith("v_accvgpr_read"):
                assert nops >= 2, (name, s)
                reads += 1
            elif s.startswith("v_accvgpr_mov"):
                assert not mfma_in_block, (name, s)
        assert reads > 0, name


def test_main_loop_mfma_operands_have_fixed_register_classes(gemm_asm):
    """Accumulators in AGPRs, fragments in VGPRs, for every MFMA of every variant."""
    for name, body in gemm_asm.items():
        for s in _instructions(body):
            if s.startswith("v_mfma_f32_16x16x32_"):
                half = "gemm_f16_" in name or "gemm_backward_kernelILb1" in name   # <HALF, ...>
                assert s.split()[0].endswith("_f16" if half else "_bf16"), (name, s)
                ops = [o.strip() for o in s.split(None, 1)[1].split(",")]
                assert ops[0].startswith("a[") and ops[3].startswith("a[") and ops[0] == ops[3], (name, s)
                assert ops[1].startswith("v[") and ops[2].startswith("v["), (name, s)


_ASM_CACHE = {}


def _device_asm(tmp_path_factory, name):
    if name in _ASM_CACHE:
        return _ASM_CACHE[name]
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("asm") / (name + ".s")
    src = os.path.join(ROOT, "axonn_amd", "csrc", name + ".hip")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.dirname(src),
           "--cuda-device-only", "-S", src, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=900)
    text = out.read_text()
    kernels = {}
    for m in re.finditer(r"^(_ZN\S+):\s", text, re.M):
        end = text.find(".end_amdhsa_kernel", m.end())
        if end > 0 and ".amdhsa_kernel" in text[m.end():end]:
            kernels[m.group(1)] = text[m.end():end]
    _ASM_CACHE[name] = kernels
    return kernels


@pytest.mark.parametrize("source", ["stream_probe", "embedding"])
def test_hand_written_stores_are_followed_by_their_wait_states(tmp_path_factory, source):
    """A store of more than 8 bytes needs wait states before its data registers are written
    again.  The compiler inserts them for its own stores, not for a store inside an asm
    statement: each of those carries its own s_nop."""
    kernels = _device_asm(tmp_path_factory, source)
    seen = 0
    for name, body in kernels.items():
        ins = _instructions(body)
        for i, s_ in enumerate(ins):
            if s_.startswith("global_store_dwordx4") and "sc1 nt" in s_:
                # (only the asm statements write "sc1 nt"; the compiler prints "nt sc1")
                seen += 1
                assert ins[i + 1].startswith("s_nop"), (name, s_, ins[i + 1])
    assert seen > 0, source


def test_update_kernel_streams_through_buffer_accesses_without_scratch(tmp_path_factory):
    """The optimizer's update kernel: no spills, every streaming access a buffer access with
    its cache policy (loads nt, stores nt sc1), all loads of the vector path ahead of the
    first store."""
    kernels = {k: v for k, v in _device_asm(tmp_path_factory, "optim").items() if "mt_adam_kernel" in k}
    assert len(kernels) == 18, sorted(kernels)   # 3 gradient types x (no copy, bf16, fp16) x with/without scan result
    for name, body in kernels.items():
        assert re.search(r"\.amdhsa_private_segment_fixed_size 0\b", body), name
        ins = _instructions(body)
        loads = [i for i, s_ in enumerate(ins) if s_.startswith("buffer_load_dwordx")]
        stores = [i for i, s_ in enumerate(ins) if s_.startswith("buffer_store_dwordx")]
        assert len(loads) == 4 and len(stores) in (3, 4), (name, len(loads), len(stores))
        assert max(loads) < min(stores), name
        assert all(ins[i].endswith(" nt") for i in loads), name
        assert all(ins[i].endswith(" nt sc1") for i in stores), name
