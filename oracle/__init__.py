"""CPU oracle of the LSTM forward + BPTT path -- test infrastructure, never imported by the product.

`oracle/lstm_oracle.c` is the restatement (double precision, PyTorch layouts); this module loads it
through ctypes and exposes numpy-in / numpy-out helpers.  Allowed importers: tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py.
"""
from .lstm_oracle import (build, forward, backward, pack_weights_v1, checkpoints, chunk_steps, round_fp16,
                          FLAG_FP16_OPERANDS, FLAG_FP16_FEEDBACK, FLAG_FP16_OUTPUT, FLAG_FP16_DG)
