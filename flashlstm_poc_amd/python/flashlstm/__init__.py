"""`flashlstm`: Python surface of the MI355X streaming LSTM (drop-in for the reference package).

Exports the same four names as the reference's flashlstm_v2/python/flashlstm/__init__.py:3-11: the
two raw-pointer extension functions and the autograd-aware wrappers built on them.
"""
from ._flashlstm import streaming_lstm_backward, streaming_lstm_forward
from .streaming_lstm import GateCache, StreamingLSTM, streaming_lstm

__all__ = [
    "streaming_lstm_forward",
    "streaming_lstm_backward",
    "streaming_lstm",
    "StreamingLSTM",
]
