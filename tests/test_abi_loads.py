"""CPU check: the C ABI library loads and exports every symbol include/neura_hip.h declares."""
import ctypes
import os
import re

from neura_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "neura_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nh_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_lists():
    assert declared_symbols() == sorted(_abi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    held = ctypes.CDLL(_abi.LIBRARY)  # loading touches no GPU
    for name in declared_symbols():
        assert hasattr(held, name), name


def test_error_message_starts_empty_and_open_fails_loudly_without_a_gpu():
    lib = _abi.library()
    assert lib.nh_last_error() is not None
    import torch  # device probe only

    if not torch.cuda.is_available():
        assert not lib.nh_open(0)
        assert b"device" in lib.nh_last_error().lower()
