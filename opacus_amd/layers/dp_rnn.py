"""RNN, GRU and LSTM built from ``RNNLinear`` so that per-sample gradients can be taken.

Mirror of opacus/layers/dp_rnn.py: ``DPRNN``, ``DPGRU``, ``DPLSTM`` are drop-in replacements
of ``torch.nn.RNN/GRU/LSTM`` (same arguments, outputs, parameter names and state dict; no
``proj_size``), written as explicit time loops over cells whose only parameters sit in two
``RNNLinear`` layers, ``ih`` and ``hh``, where the grad-sample hooks can see them.

Shaped for the per-sample-gradient kernels rather than as a transcription:

* the input projection does not depend on the recurrence, so ``ih`` is applied once to the
  whole ``[B, T, D]`` sequence of a layer and direction. Its per-sample gradient is then one
  contraction over T on the matrix cores instead of T rank-one products summed in memory;
* ``hh`` runs once per time step; the grad-sample module stacks those uses
  (``RNNLinear.stack_uses``) and contracts them over time in one launch as well;
* a ``PackedSequence`` is processed as a padded batch with a per-step mask: finished
  sequences keep their state and receive zero backprops, which gives the outputs and
  gradients of step-wise shrinking batches without ragged shapes. The padded batch is in the
  caller's sample order, not the packed (sorted by length) one, so row i of every per-sample
  gradient belongs to the same sample i as in the layers around the RNN. (The reference runs
  its cells in sorted order, so with ``enforce_sorted=False`` its RNN gradients are permuted
  against the other layers' and the per-sample norm mixes samples.)
"""

from __future__ import annotations

import math
import numbers
import warnings
from typing import List, Optional, Tuple, Type, Union

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn.utils.rnn import PackedSequence

from .param_rename import RenameParamsMixin


def apply_permutation(tensor: Tensor, dim: int, permutation: Optional[Tensor]) -> Tensor:
    """``tensor`` reordered along ``dim``; unchanged when ``permutation`` is None (dp_rnn.py:30-36)."""
    if permutation is None:
        return tensor
    return tensor.index_select(dim, permutation)


class RNNLinear(nn.Linear):
    """``nn.Linear`` for layers applied many times per forward pass (dp_rnn.py:39-53): its
    per-sample gradients over the uses of one pass are summed, and its batch dimension is
    always the first. ``max_batch_len`` is the batch size the per-sample gradient is laid
    out for when single uses see fewer samples."""

    max_batch_len: int
    # read by the grad-sample hooks: gather all uses of one backward pass and contract them
    # in one sampler call
    stack_uses = True

    def __init__(self, in_features: int, out_features: int, bias: bool = True):
        super().__init__(in_features, out_features, bias)


class DPRNNCellBase(nn.Module):
    """Two ``RNNLinear`` maps, input to gates (``ih``) and hidden state to gates (``hh``),
    each ``num_chunks * hidden_size`` wide (dp_rnn.py:56-79)."""

    has_cell_state: bool = False

    def __init__(self, input_size: int, hidden_size: int, bias: bool, num_chunks: int) -> None:
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.bias = bias
        self.ih = RNNLinear(input_size, num_chunks * hidden_size, bias)
        self.hh = RNNLinear(hidden_size, num_chunks * hidden_size, bias)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        stdv = 1.0 / math.sqrt(self.hidden_size)
        for weight in self.parameters():
            nn.init.uniform_(weight, -stdv, stdv)

    def set_max_batch_length(self, max_batch_length: int) -> None:
        self.ih.max_batch_len = max_batch_length
        self.hh.max_batch_len = max_batch_length

    def _zero_state(self, like: Tensor) -> Tensor:
        return torch.zeros(like.shape[0], self.hidden_size, dtype=like.dtype, device=like.device)

    def step(self, gates_x: Tensor, h_prev: Tensor, c_prev: Optional[Tensor]) -> Tuple[Tensor, Optional[Tensor]]:
        """One time step from the already projected input ``gates_x = ih(x_t)``."""
        raise NotImplementedError

    def _single(self, input: Tensor, h_prev: Tensor, c_prev: Optional[Tensor], batch_size_t: Optional[int]):
        if batch_size_t is not None:
            h_prev = h_prev[:batch_size_t, :]
            c_prev = None if c_prev is None else c_prev[:batch_size_t, :]
        return self.step(self.ih(input), h_prev, c_prev)


class DPRNNCell(DPRNNCellBase):
    """Elman cell, ``h' = act(W_ih x + b_ih + W_hh h + b_hh)`` with tanh or ReLU (dp_rnn.py:82-118)."""

    def __init__(self, input_size: int, hidden_size: int, bias: bool, nonlinearity: str = "tanh") -> None:
        super().__init__(input_size, hidden_size, bias, num_chunks=1)
        if nonlinearity not in ("tanh", "relu"):
            raise ValueError(f"Unsupported nonlinearity: {nonlinearity}")
        self.nonlinearity = nonlinearity

    def step(self, gates_x, h_prev, c_prev=None):
        pre = gates_x + self.hh(h_prev)
        return (torch.tanh(pre) if self.nonlinearity == "tanh" else torch.relu(pre)), None

    def forward(self, input: Tensor, hx: Optional[Tensor] = None, batch_size_t: Optional[int] = None) -> Tensor:
        h_prev = self._zero_state(input) if hx is None else hx
        return self._single(input, h_prev, None, batch_size_t)[0]


class DPGRUCell(DPRNNCellBase):
    """GRU cell with torch's gate order (reset, update, new) (dp_rnn.py:121-155)."""

    def __init__(self, input_size: int, hidden_size: int, bias: bool) -> None:
        super().__init__(input_size, hidden_size, bias, num_chunks=3)

    def step(self, gates_x, h_prev, c_prev=None):
        xr, xz, xn = torch.split(gates_x, self.hidden_size, 1)
        hr, hz, hn = torch.split(self.hh(h_prev), self.hidden_size, 1)
        r = torch.sigmoid(xr + hr)
        z = torch.sigmoid(xz + hz)
        n = torch.tanh(xn + r * hn)
        return (1 - z) * n + z * h_prev, None

    def forward(self, input: Tensor, hx: Optional[Tensor] = None, batch_size_t: Optional[int] = None) -> Tensor:
        h_prev = self._zero_state(input) if hx is None else hx
        return self._single(input, h_prev, None, batch_size_t)[0]


class DPLSTMCell(DPRNNCellBase):
    """LSTM cell with torch's gate order (input, forget, cell, output) (dp_rnn.py:158-207)."""

    has_cell_state = True

    def __init__(self, input_size: int, hidden_size: int, bias: bool) -> None:
        super().__init__(input_size, hidden_size, bias, num_chunks=4)

    def step(self, gates_x, h_prev, c_prev):
        i, f, g, o = torch.split(gates_x + self.hh(h_prev), self.hidden_size, 1)
        c = torch.sigmoid(f) * c_prev + torch.sigmoid(i) * torch.tanh(g)
        return torch.sigmoid(o) * torch.tanh(c), c

    def forward(
        self, input: Tensor, hx: Optional[Tuple[Tensor, Tensor]] = None, batch_size_t: Optional[int] = None
    ) -> Tuple[Tensor, Tensor]:
        if hx is None:
            zeros = self._zero_state(input)
            hx = (zeros, zeros)
        return self._single(input, hx[0], hx[1], batch_size_t)


RNN_CELL_TYPES = {
    "RNN_TANH": (DPRNNCell, {"nonlinearity": "tanh"}),
    "RNN_RELU": (DPRNNCell, {"nonlinearity": "relu"}),
    "GRU": (DPGRUCell, {}),
    "LSTM": (DPLSTMCell, {}),
}


class DPRNNBase(RenameParamsMixin, nn.Module):
    """Multi-layer, optionally bidirectional sequence model over an abstract cell
    (dp_rnn.py:218-634). Inputs and outputs as ``torch.nn.RNNBase``: a ``[T, B, D]`` tensor
    (``[B, T, D]`` with ``batch_first``) or a ``PackedSequence``, and initial states
    ``[layers * directions, B, H]``."""

    # the grad-sample hooks go to the RNNLinear children; the parameters registered on this
    # module are their aliases under torch's names
    grad_sample_through_children = True

    def __init__(
        self,
        mode: Union[str, Type[DPRNNCellBase]],
        input_size: int,
        hidden_size: int,
        num_layers: int = 1,
        bias: bool = True,
        batch_first: bool = False,
        dropout: float = 0.0,
        bidirectional: bool = False,
        proj_size: int = 0,
        cell_params: Optional[dict] = None,
    ) -> None:
        super().__init__()
        self.cell_params = {}
        if isinstance(mode, str):
            if mode not in RNN_CELL_TYPES:
                raise ValueError(f"Invalid RNN mode '{mode}', available options: {list(RNN_CELL_TYPES.keys())}")
            self.cell_type, default_params = RNN_CELL_TYPES[mode]
            self.cell_params.update(default_params)
        else:
            self.cell_type = mode
        if cell_params is not None:
            self.cell_params.update(cell_params)
        self.has_cell_state = self.cell_type.has_cell_state

        self.input_size = input_size
        self.hidden_size = hidden_size
        self.num_layers = num_layers
        self.bias = bias
        self.batch_first = batch_first
        if not isinstance(dropout, numbers.Number) or not 0 <= dropout <= 1 or isinstance(dropout, bool):
            raise ValueError(
                "dropout should be a number in range [0, 1] representing the probability of an element being zeroed"
            )
        self.dropout = float(dropout)
        self.bidirectional = bidirectional
        self.proj_size = proj_size
        self.num_directions = 2 if bidirectional else 1
        if dropout > 0 and num_layers == 1:
            warnings.warn(
                "dropout option adds dropout after all but last recurrent layer, so non-zero dropout expects "
                f"num_layers greater than 1, but got dropout={dropout} and num_layers={num_layers}"
            )
        if proj_size > 0:
            raise NotImplementedError("proj_size > 0 is not supported")
        if proj_size < 0:
            raise ValueError("proj_size should be a positive integer or zero to disable projections")
        if proj_size >= hidden_size:
            raise ValueError("proj_size has to be smaller than hidden_size")
        self.dropout_layer = nn.Dropout(dropout) if dropout > 0 else None
        self.cells = self.initialize_cells()

    # ---- construction ----------------------------------------------------------------------
    def initialize_cells(self) -> List[DPRNNCellBase]:
        """Cells ``l{k}`` and ``l{k}_reverse``; their parameters appear as
        ``weight_ih_l{k}[_reverse]`` etc., the names of ``torch.nn.RNNBase`` (dp_rnn.py:604-634)."""
        cells, rename_map = [], {}
        for layer in range(self.num_layers):
            for direction in range(self.num_directions):
                in_size = self.input_size if layer == 0 else self.hidden_size * self.num_directions
                cell = self.cell_type(in_size, self.hidden_size, bias=self.bias, **self.cell_params)
                cells.append(cell)
                name = f"l{layer}" + ("_reverse" if direction == 1 else "")
                setattr(self, name, cell)
                for kind in ["weight"] + (["bias"] if self.bias else []):
                    for matrix in ("ih", "hh"):
                        rename_map[f"{name}.{matrix}.{kind}"] = f"{kind}_{matrix}_{name}"
        self.set_rename_map(rename_map)
        return cells

    def iterate_layers(self, *args):
        """Yields ``(layer, ((direction, (arg[layer, direction] for arg in args)), ...))``
        for lists laid out ``[layers * directions]`` (dp_rnn.py:571-602)."""
        for layer in range(self.num_layers):
            yield layer, (
                (direction, tuple(arg[self.num_directions * layer + direction] for arg in args))
                for direction in range(self.num_directions)
            )

    # ---- forward ----------------------------------------------------------------------------
    def forward(
        self,
        input: Union[Tensor, PackedSequence],
        state_init: Optional[Union[Tensor, Tuple[Tensor, Tensor]]] = None,
    ) -> Tuple[Union[Tensor, PackedSequence], Union[Tensor, Tuple[Tensor, Tensor]]]:
        is_packed = isinstance(input, PackedSequence)
        if is_packed:
            data, batch_sizes, sorted_indices, unsorted_indices = input
            seq_length, max_batch = len(batch_sizes), int(batch_sizes[0])
            # live[t, b]: sample b (packed order) still has a step t
            live = torch.arange(max_batch).unsqueeze(0) < batch_sizes.unsqueeze(1)  # [T, B] on the host
            live = live.to(data.device)
            x = data.new_zeros(seq_length, max_batch, data.shape[-1])
            x[live] = data  # row-major over (t, b) is the packed order
            live_packed = live
            if unsorted_indices is not None:  # back to the caller's sample order
                x = x.index_select(1, unsorted_indices)
                live = live.index_select(1, unsorted_indices)
            for cell in self.cells:
                cell.set_max_batch_length(max_batch)
        else:
            sorted_indices = unsorted_indices = live = live_packed = None
            x = input.transpose(0, 1) if self.batch_first else input  # [T, B, D]
            seq_length, max_batch = x.shape[0], x.shape[1]
        dtype, device = x.dtype, x.device

        if self.has_cell_state:
            h_0s, c_0s = state_init or (None, None)
        else:
            h_0s, c_0s = state_init, None
        n_states = self.num_layers * self.num_directions
        if h_0s is None:
            h_0s = torch.zeros(n_states, max_batch, self.hidden_size, dtype=dtype, device=device)
        if self.has_cell_state:
            if c_0s is None:
                c_0s = torch.zeros(n_states, max_batch, self.hidden_size, dtype=dtype, device=device)
        else:
            c_0s = [None] * n_states

        hs, cs = [], []
        output = x
        for _layer, directions in self.iterate_layers(self.cells, h_0s, c_0s):
            outs = []
            for direction, (cell, h0, c0) in directions:
                out, h, c = self.forward_layer(output, h0, c0, cell=cell, live=live, reverse_layer=(direction == 1))
                outs.append(out)
                hs.append(h)
                cs.append(c)
            output = outs[0] if len(outs) == 1 else torch.cat(outs, dim=2)  # [T, B, P*H]

        if is_packed:
            output = apply_permutation(output, 1, sorted_indices)
            output = PackedSequence(output[live_packed], batch_sizes, sorted_indices, unsorted_indices)
        elif self.batch_first:
            output = output.transpose(0, 1)
        hs = torch.stack(hs, dim=0)
        if self.has_cell_state:
            return output, (hs, torch.stack(cs, dim=0))
        return output, hs

    def forward_layer(
        self,
        x: Tensor,
        h_0: Tensor,
        c_0: Optional[Tensor],
        *,
        cell: DPRNNCellBase,
        live: Optional[Tensor],
        reverse_layer: bool,
    ) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
        """One layer in one direction over ``x`` ``[T, B, D]``: returns the outputs
        ``[T, B, H]`` in input order and the last states ``[B, H]``. ``live`` ``[T, B]`` marks
        the steps that exist; elsewhere the state is carried over and the output is zero."""
        T = x.shape[0]
        # all input projections of the layer in one call, batch first for the sampler
        gates_x = cell.ih(x.transpose(0, 1))  # [B, T, chunks * H]
        h, c = h_0, c_0
        outs: List[Optional[Tensor]] = [None] * T
        for t in (range(T - 1, -1, -1) if reverse_layer else range(T)):
            h_new, c_new = cell.step(gates_x[:, t], h, c)
            if self.dropout_layer is not None:
                # as the reference: on the state that is both emitted and carried on (dp_rnn.py:541-542)
                h_new = self.dropout_layer(h_new)
            if live is not None:
                m = live[t].unsqueeze(1)
                h = torch.where(m, h_new, h)
                if c_new is not None:
                    c = torch.where(m, c_new, c)
                outs[t] = h_new * m
            else:
                h, c = h_new, c_new
                outs[t] = h_new
        return torch.stack(outs, dim=0), h, c


class DPRNN(DPRNNBase):
    """Drop-in replacement of ``torch.nn.RNN`` (dp_rnn.py:637-670)."""

    def __init__(
        self,
        input_size: int,
        hidden_size: int,
        num_layers: int = 1,
        bias: bool = True,
        batch_first: bool = False,
        dropout: float = 0,
        bidirectional: bool = False,
        proj_size: int = 0,
        nonlinearity: str = "tanh",
    ) -> None:
        super().__init__(
            DPRNNCell, input_size, hidden_size, num_layers=num_layers, bias=bias, batch_first=batch_first,
            dropout=dropout, bidirectional=bidirectional, proj_size=proj_size, cell_params={"nonlinearity": nonlinearity},
        )


class DPGRU(DPRNNBase):
    """Drop-in replacement of ``torch.nn.GRU`` (dp_rnn.py:673-703)."""

    def __init__(
        self,
        input_size: int,
        hidden_size: int,
        num_layers: int = 1,
        bias: bool = True,
        batch_first: bool = False,
        dropout: float = 0,
        bidirectional: bool = False,
        proj_size: int = 0,
    ) -> None:
        super().__init__(
            DPGRUCell, input_size, hidden_size, num_layers=num_layers, bias=bias, batch_first=batch_first,
            dropout=dropout, bidirectional=bidirectional, proj_size=proj_size,
        )


class DPLSTM(DPRNNBase):
    """Drop-in replacement of ``torch.nn.LSTM`` (dp_rnn.py:706-736)."""

    def __init__(
        self,
        input_size: int,
        hidden_size: int,
        num_layers: int = 1,
        bias: bool = True,
        batch_first: bool = False,
        dropout: float = 0,
        bidirectional: bool = False,
        proj_size: int = 0,
    ) -> None:
        super().__init__(
            DPLSTMCell, input_size, hidden_size, num_layers=num_layers, bias=bias, batch_first=batch_first,
            dropout=dropout, bidirectional=bidirectional, proj_size=proj_size,
        )
