"""MI355X-native LSTM forward + BPTT (gfx950 HIP kernels behind a C ABI).

`LstmCore` drives the device-resident core (`include/flashlstm/lstm_core.h`) from torch tensors;
the drop-in `flashlstm` Python package of the streaming surface lives in `flashlstm_poc_amd/python`.
"""
from .core import LstmCore, load_library, library_path, LibraryMissing, add_flashlstm_to_path
from .stack import LstmStack, StackedLSTM

__all__ = ["LstmCore", "LstmStack", "StackedLSTM", "load_library", "library_path", "LibraryMissing", "add_flashlstm_to_path"]
