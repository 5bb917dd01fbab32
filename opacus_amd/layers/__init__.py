from .dp_multihead_attention import DPMultiheadAttention, SequenceBias
from .dp_rnn import DPGRU, DPLSTM, DPRNN, RNNLinear
from .param_rename import RenameParamsMixin

__all__ = ["DPRNN", "DPGRU", "DPLSTM", "DPMultiheadAttention", "RNNLinear", "RenameParamsMixin", "SequenceBias"]
