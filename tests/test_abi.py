"""The C-ABI library loads and exports every entry point include/jetfire_hip.h declares (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header="jetfire_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jf_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = _declared()
    assert len(names) >= 16
    lib = ctypes.CDLL(os.path.join(ROOT, "jetfire-int8training_amd", "libjetfire_hip.so"))
    for n in names:
        assert hasattr(lib, n), n


def test_binding_lists_every_symbol(jf):
    assert sorted(jf.EXPORTS) == _declared()


def test_measurement_library_is_separate(jf):
    """The measurement aids live in their own library and header: the product library exports only what jetfire_hip.h
    declares (the reference's interfaces and the allocation-free entry point)."""
    names = _declared("jetfire_prof.h")
    assert sorted(jf.PROF_EXPORTS) == names and len(names) == 3
    prof = ctypes.CDLL(os.path.join(ROOT, "jetfire-int8training_amd", "libjetfire_prof.so"))
    main = ctypes.CDLL(os.path.join(ROOT, "jetfire-int8training_amd", "libjetfire_hip.so"))
    for n in names:
        assert hasattr(prof, n), n
        assert not hasattr(main, n), f"{n} belongs to the measurement library"


def test_argument_errors_without_gpu(jf):
    L = jf.lib()
    assert L.jf_igemm_s32(None, None, None, 32, 32, 32, 0, None, 0, None) == -1
    assert b"NULL" in L.jf_error_string(-1)
    assert b"multiple of 32" in L.jf_error_string(-2)
    assert L.jf_igemm_workspace_bytes(64, 96, 128, 1) == 0      # a [K,N] operand is read in place
    assert L.jf_igemm_workspace_bytes(64, 96, 128, 0) == 0
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 15) & ~15
    assert L.jf_igemm_s32(p, p, p, 48, 32, 32, 0, None, 0, None) == -2          # 48 is not a multiple of 32
    assert L.jf_igemm_s32(p, p, p, 32, 32, 32, 7, None, 0, None) == -3          # unknown layout
    assert L.jf_igemm_s32(p + 1, p, p, 32, 32, 32, 0, None, 0, None) == -4      # misaligned
    assert L.jf_quantize(p, 9, 32, 32, p, p, None, 0, 0, 0, 0, 0.0, None) == -3
    # scale arrays: natural alignment of their element type (2 bytes for binary16, 4 for binary32)
    q_args = (None, None, p, p, 32, 32, 32, 0)
    assert L.jf_igemm_block_q(p, p, p + 2, p, *q_args, 1, 0, 0, 0, 0, 0, None, 0, None) == -4
    assert L.jf_igemm_block_q(p, p, p + 1, p, *q_args, 0, 0, 0, 0, 0, 0, None, 0, None) == -4
    import torch
    if not torch.cuda.is_available():
        # binary16 scales at an even address pass the alignment check; with no device the call is then refused by name.
        # (Only without a GPU: p is host memory, and with a device present valid arguments would launch a kernel on it.)
        assert L.jf_igemm_block_q(p, p, p + 2, p, *q_args, 0, 0, 0, 0, 0, 0, None, 0, None) == -6
        # valid arguments, but no gfx950 device to run on: refused by name, nothing is launched
        assert L.jf_igemm_s32(p, p, p, 32, 32, 32, 0, None, 0, None) == -6
        assert L.jf_quantize(p, 1, 32, 32, p, p, None, 0, 0, 0, 0, 0.0, None) == -6
        assert b"gfx950" in L.jf_error_string(-6)
    assert L.jf_gelu_fwd(p, p, 32, 32, 0, 5, 0.0, p, p, None) == -3
    # the allocation-free weight-gradient entry point refuses a K split that does not fit its built-in scratch buffer
    # (16 parts of 1600 x 1600 fp32 = 164 MB) before it touches the device
    assert L.jf_igemm_block_fp_noalloc(p, p, p, p, p, 1600, 1600, 8192, 0, 1, 1, 0, 0, 1, 16, None) == -8
    assert b"scratch" in L.jf_error_string(-8)
