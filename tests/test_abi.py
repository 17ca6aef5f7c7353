"""The C-ABI library loads and exports every symbol the public header declares (no GPU calls)."""
import os
import re

import pytest

from gllm_amd import backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "gllm_hip_quant.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gllmq_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    assert _declared_symbols() == sorted(backend.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(backend.LIB_PATH):
        pytest.fail(f"{backend.LIB_PATH} missing: run python -m gllm_amd.build")
    lib = backend.load_library()
    for name in _declared_symbols():
        assert hasattr(lib, name), name


def test_format_constants_through_the_abi():
    lib = backend.load_library()
    # src/loader/gguf/types.rs:594-629,998-999,1548,1941-1948,1971-1972
    assert [lib.gllmq_block_size(t) for t in (8, 12, 13, 14)] == [32, 256, 256, 256]
    assert [lib.gllmq_block_bytes(t) for t in (8, 12, 13, 14)] == [34, 144, 176, 210]
    assert lib.gllmq_block_size(2) == 0 and lib.gllmq_block_bytes(15) == 0
    assert lib.gllmq_row_bytes(8, 33) == 68 and lib.gllmq_row_bytes(12, 256) == 144
    assert lib.gllmq_row_bytes(12, 4096) * 14336 == 33_030_144
    assert lib.gllmq_row_bytes(14, 4096) * 14336 == 48_168_960
    assert lib.gllmq_status_string(1) == b"unimplemented"
    assert lib.gllmq_version().startswith(b"gllm_hip_quant")


def test_python_mirror_of_the_constants():
    from gllm_amd import ggml
    assert ggml.tensor_nbytes(ggml.GgmlDType.Q4_K, [256, 4]) == 576
    assert ggml.tensor_nbytes(ggml.GgmlDType.Q6_K, [256, 4]) == 840
    assert ggml.tensor_nbytes(ggml.GgmlDType.Q8_0, [33]) == 68
    assert ggml.QuantType.Q4K.block_bytes() == 144 and ggml.QuantType.Q6K.ggml_dtype == 14


def test_backend_refuses_to_run_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(backend.HipError):
        backend.HipBackend()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; any other --gpus value exits with a message, before touching a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, timeout=60)
    assert r.returncode == 2
    assert b"one GPU" in r.stderr
    assert r.stdout.strip() == b""
