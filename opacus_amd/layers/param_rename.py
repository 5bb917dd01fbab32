"""Modules whose parameters are listed and saved under other names than their attribute paths.

Mirror of opacus/layers/param_rename.py (``RenameParamsMixin``): ``DPLSTM`` keeps its
weights inside per-layer cell submodules, yet ``named_parameters()`` and ``state_dict()``
must read like ``torch.nn.LSTM``'s (``weight_ih_l0`` ...), so that a trained model loads into
the stock module.

How it is done here: the renamed parameter is also registered on the mixin's own module under
the new name. ``named_parameters()`` walks a module's own parameters before its children and
drops repeats, so the new name is the one listed. A state-dict hook removes the old keys on
save and a load pre-hook copies each new key to its old twin on load, so strict loading sees
every key it expects.
"""

from __future__ import annotations

from typing import Dict

import torch.nn as nn


def _drop_old_keys(module, state_dict, prefix, _local_metadata):
    for old in module.old_to_new:
        state_dict.pop(prefix + old, None)
    return state_dict


def _add_old_keys(module, state_dict, prefix, *_):
    for old, new in module.old_to_new.items():
        if prefix + new in state_dict and prefix + old not in state_dict:
            state_dict[prefix + old] = state_dict[prefix + new]


class RenameParamsMixin:
    """``set_rename_map({"cell.w": "w_cell"})`` after the parameters exist; the map must be
    one to one."""

    def set_rename_map(self, rename_map: Dict[str, str]) -> None:
        if len(set(rename_map.values())) != len(rename_map):
            raise ValueError("rename_map must be a one-to-one mapping")
        self.old_to_new = dict(rename_map)
        self.new_to_old = {v: k for k, v in rename_map.items()}
        params = dict(nn.Module.named_parameters(self))
        for old, new in self.old_to_new.items():
            if old in params:
                self.register_parameter(new, params[old])
        self._register_state_dict_hook(_drop_old_keys)
        self.register_load_state_dict_pre_hook(_add_old_keys)
