from .dp_rnn import DPGRU, DPLSTM, DPRNN, RNNLinear
from .param_rename import RenameParamsMixin

__all__ = ["DPRNN", "DPGRU", "DPLSTM", "RNNLinear", "RenameParamsMixin"]
