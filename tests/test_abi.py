"""CPU-side checks of the drop-in boundary: the shared library loads, exports every function the
public headers declare, and the Python surface rejects bad arguments before touching a GPU."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = ["include/flashlstm/lstm_api.h", "include/flashlstm/lstm_core.h", "include/flashlstm_v2/lstm.hpp"]


def _declared_c_functions(path):
    text = open(os.path.join(ROOT, path)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    # every C entry point carries the lstm_ / flstm_ prefix (the C++ overloads in namespace flstm do not)
    return set(re.findall(r"\b((?:lstm|flstm)_\w+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    from flashlstm_poc_amd import library_path
    lib = ctypes.CDLL(library_path())
    declared = set()
    for h in HEADERS:
        declared |= _declared_c_functions(h)
    expected = {"lstm_create_buffers", "lstm_destroy_buffers", "lstm_set_execution_mode", "lstm_pack_weights",
                "lstm_forward", "lstm_backward", "flstm_StreamingLstmForward", "flstm_StreamingLstmBackward",
                "flstm_core_create", "flstm_core_forward", "flstm_core_backward"}
    assert expected <= declared, expected - declared
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in a header but not exported"


def test_split_count_rule_of_the_weight_gradient_gemm():
    # A pure function of the sizes: blocks of 32 tiles x splits are dealt to the 8 XCDs in rounds, a round runs
    # K / splits, every work item costs a fixed extra.  Pinned on cases whose answer follows from counting rounds.
    from flashlstm_poc_amd import library_path
    lib = ctypes.CDLL(library_path())
    f = lib.flstm_gemm_tn_auto_splits
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int]
    assert f(4096, 2048, 262144, 64) == 2      # 128 tiles = 4 blocks: one split leaves half the XCDs idle, two fill them
    assert f(8192, 4096, 524288, 64) == 1      # 512 tiles = 16 blocks: two full rounds already
    assert f(8192, 2560, 524288, 64) == 4      # 320 tiles = 10 blocks: 2 rounds at one split, 5 full rounds at four
    assert f(256, 256, 1 << 20, 64) == 8       # one block: a split per XCD, more only adds partial tiles
    assert f(256, 256, 1 << 20, 3) == 3        # capped by the caller
    assert f(4096, 2048, 64, 64) == 1          # a single 64-row slab cannot be split
    assert f(0, 2048, 4096, 8) == 1 and f(4096, 2048, 4096, 0) == 1


def test_v1_enum_values_and_handle_layout():
    text = open(os.path.join(ROOT, "include/flashlstm/lstm_api.h")).read()
    assert re.search(r"LSTM_COMPUTE_PRECISION_FP16_ACC32\s*=\s*0", text)
    assert re.search(r"LSTM_COMPUTE_PRECISION_FP16_ACC16\s*=\s*1", text)
    assert re.search(r"LSTM_EXECUTION_MODE_IMMEDIATE\s*=\s*0", text)
    assert re.search(r"LSTM_EXECUTION_MODE_GRAPH\s*=\s*1", text)
    assert re.search(r"typedef struct lstm_buffers \{\s*void\* impl;\s*\} lstm_buffers;", text)


def test_v1_argument_validation_without_gpu():
    # null handle / null impl are rejected with 1 (= hipErrorInvalidValue) before any device work
    from flashlstm_poc_amd import library_path
    lib = ctypes.CDLL(library_path())

    class Buffers(ctypes.Structure):
        _fields_ = [("impl", ctypes.c_void_p)]

    b = Buffers(None)
    assert lib.lstm_destroy_buffers(None) == 1
    assert lib.lstm_set_execution_mode(ctypes.byref(b), 1) == 1
    assert lib.lstm_pack_weights(0, None, None, ctypes.c_size_t(4), ctypes.c_size_t(4), ctypes.byref(b)) == 1
    assert lib.lstm_create_buffers(7, ctypes.c_size_t(1), ctypes.c_size_t(1), ctypes.c_size_t(1), ctypes.c_size_t(1),
                                   0, ctypes.byref(b)) == 1
    assert b.impl is None


def test_core_argument_validation_without_gpu():
    from flashlstm_poc_amd import load_library
    lib = load_library()
    h = ctypes.c_void_p()
    assert lib.flstm_core_create(0, 4, 4, ctypes.byref(h)) == 1
    assert lib.flstm_core_create(4, 4, 4, None) == 1
    assert lib.flstm_core_destroy(None) == 1
    assert lib.flstm_core_get_info(None, b"fallbacks") == -1


def test_extension_module_signature_checks():
    import flashlstm
    assert set(flashlstm.__all__) == {"streaming_lstm_forward", "streaming_lstm_backward", "streaming_lstm",
                                      "StreamingLSTM"}
    with pytest.raises(TypeError):
        flashlstm.streaming_lstm_forward(1, 2, 3)
    with pytest.raises(TypeError):
        flashlstm.streaming_lstm_backward(*([0] * 29))
    with pytest.raises(TypeError):
        flashlstm.streaming_lstm_forward(*([0.5] * 22))
    # zero sizes are a silent no-op (reference lstm_forward.cu:493-495): safe without a GPU
    assert flashlstm.streaming_lstm_forward(*([0] * 22)) is None
    assert flashlstm.streaming_lstm_backward(*([0] * 30)) is None


def test_python_surface_rejects_bad_host_tensors():
    from flashlstm.streaming_lstm import _StreamingLSTMFunction, _cache_dtype_code, GateCache
    assert _cache_dtype_code(torch.float32) == 0 and _cache_dtype_code(torch.float16) == 1
    with pytest.raises(ValueError, match="gate cache dtype"):
        _cache_dtype_code(torch.bfloat16)
    assert GateCache._fields == ("h", "c")
    w = torch.zeros(8, 3)
    args = (None, None, w, w, w, w, 1, (torch.float32, torch.float32))
    with pytest.raises(ValueError, match="pinned"):
        _StreamingLSTMFunction.apply(torch.zeros(4, 2, 3, dtype=torch.float16), *args)
    with pytest.raises(ValueError, match="dtype"):
        _StreamingLSTMFunction.apply(torch.zeros(4, 2, 3, dtype=torch.float32), *args)
