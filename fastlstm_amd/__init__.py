"""MI355X-native LSTM forward/backward behind the FastLSTM Python interface."""
from .lstm import (FastLSTM, PersistentLSTMfn, PersistentLSTMStatefn, Wgrad, lstm_persistent_bwd,  # noqa: F401
                   lstm_persistent_fwd, pending_status)
