"""Falcon-7B MLP: dense_h_to_4h with fused GELU, then dense_4h_to_h (models/demos/falcon7b/tt/falcon_mlp.py:13-80).

Weights are the transposed torch weights ([in, out]) as BFLOAT8_B tiles on the device
(models/demos/falcon7b/tt/model_config.py: DENSE_H_TO_4H_MM_WEIGHTS_DTYPE / DENSE_4H_TO_H_MM_WEIGHTS_DTYPE); the reference
reads them from its weight cache (model_utils.py get_weights_cached), here they are converted or — with tt_cache_path —
cached as tensor files of the reference's format.
"""
from __future__ import annotations

import pathlib
from typing import Optional

import torch

import tt_lib
import ttnn


def falcon_mlp_model_config(weights_dtype=None, output_dtype=None):
    """The entries of the reference's model_config that this block reads."""
    weights_dtype = weights_dtype if weights_dtype is not None else tt_lib.tensor.DataType.BFLOAT8_B
    output_dtype = output_dtype if output_dtype is not None else tt_lib.tensor.DataType.BFLOAT16
    mem = tt_lib.tensor.MemoryConfig()
    return {
        "DENSE_H_TO_4H_MM_WEIGHTS_DTYPE": weights_dtype, "DENSE_4H_TO_H_MM_WEIGHTS_DTYPE": weights_dtype,
        "DENSE_H_TO_4H_MM_WEIGHTS_MEMCFG": mem, "DENSE_4H_TO_H_MM_WEIGHTS_MEMCFG": mem,
        "DENSE_H_TO_4H_MM_OUTPUT_MEMCFG": mem, "DENSE_4H_TO_H_MM_OUTPUT_MEMCFG": mem,
        "DENSE_H_TO_4H_MM_OUTPUT_DTYPE": output_dtype, "DENSE_4H_TO_H_MM_OUTPUT_DTYPE": output_dtype,
    }


class TtFalconMLP(torch.nn.Module):
    def __init__(self, devices, state_dict, base_url, layer_num, hidden_size: int, model_config, tt_cache_path: Optional[pathlib.Path] = None):
        super().__init__()
        self.devices = list(devices)
        self.hidden_size = hidden_size
        self.model_config = model_config
        layer_name = f"{base_url}.{layer_num}"
        self.dense_h_to_4h_weights = self._weights(state_dict, f"{layer_name}.mlp.dense_h_to_4h.weight", "DENSE_H_TO_4H_MM_WEIGHTS", tt_cache_path)
        self.dense_4h_to_h_weights = self._weights(state_dict, f"{layer_name}.mlp.dense_4h_to_h.weight", "DENSE_4H_TO_H_MM_WEIGHTS", tt_cache_path)

    def _weights(self, state_dict, name, config_str, tt_cache_path):
        dtype = self.model_config[f"{config_str}_DTYPE"]
        weight = torch.transpose(state_dict[name], -2, -1).unsqueeze(0).unsqueeze(0)     # [1, 1, in, out]
        cache = None if tt_cache_path is None else pathlib.Path(tt_cache_path) / name
        return [ttnn.as_tensor(weight, dtype=dtype, layout=ttnn.TILE_LAYOUT, device=device, cache_file_name=cache) for device in self.devices]

    def forward(self, x):
        """x: one activation tensor per device, [1, 1, seq, hidden] BFLOAT16 TILE on that device; returns the same list form."""
        hidden_states = []
        for device_id in range(len(x)):
            hidden_states.append(
                tt_lib.tensor.falcon_dense_h_to_4h_matmul(
                    x[device_id], self.dense_h_to_4h_weights[device_id],
                    fused_activation=[tt_lib.tensor.FusibleActivation.GELU, True],
                    output_mem_config=self.model_config["DENSE_H_TO_4H_MM_OUTPUT_MEMCFG"],
                    output_dtype=self.model_config["DENSE_H_TO_4H_MM_OUTPUT_DTYPE"]))
            x[device_id].deallocate()
        for device_id in range(len(x)):
            hidden_states[device_id] = tt_lib.tensor.falcon_dense_4h_to_h_matmul(
                hidden_states[device_id], self.dense_4h_to_h_weights[device_id],
                output_mem_config=self.model_config["DENSE_4H_TO_H_MM_OUTPUT_MEMCFG"],
                output_dtype=self.model_config["DENSE_4H_TO_H_MM_OUTPUT_DTYPE"], packer_l1_acc=True)
        return hidden_states
