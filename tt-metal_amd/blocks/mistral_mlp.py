"""Mistral-7B MLP: down(silu(gate(x)) * up(x)) (models/demos/mistral7b/tt/mistral_mlp.py:9-82).

w1 = gate_proj, w3 = up_proj, w2 = down_proj; the reference keeps w1 and w3 in BFLOAT4_B and w2 in BFLOAT8_B or BFLOAT4_B
depending on the configuration (models/demos/mistral7b/tt/model_config.py), all as tiles through ttnn.as_tensor with a
weight cache.
"""
from __future__ import annotations

import pathlib
from typing import Optional

import torch

import ttnn


def mistral_mlp_model_config():
    """The entries of the reference's model_config that this block reads (memory configurations have no meaning here)."""
    mem = ttnn.DRAM_MEMORY_CONFIG
    return {"MLP_W_LAYOUT_TILE": ttnn.TILE_LAYOUT, "MLP_WEIGHTS_MEMCFG": mem, "FF1_OUTPUT_MEMCFG": mem, "FF2_OUTPUT_MEMCFG": mem,
            "FF3_OUTPUT_MEMCFG": mem}


class _Args:
    max_grid_size = ttnn.CoreGrid(y=8, x=8)

    @staticmethod
    def get_compute_kernel_config():
        return None


class TtMistralMLP(torch.nn.Module):
    def __init__(self, device, args, state_dict, weight_cache_path: Optional[pathlib.Path], layer_num, dtype, model_config):
        super().__init__()
        self.device = device
        self.args = args if args is not None else _Args()
        self.model_config = model_config
        base_name = f"layers.{layer_num}.feed_forward"
        torch_weight = lambda name: torch.transpose(state_dict[f"{base_name}.{name}.weight"], -2, -1)
        cache_name = lambda name: None if weight_cache_path is None else pathlib.Path(weight_cache_path) / (base_name + f".{name}")
        as_tensor = lambda name: ttnn.as_tensor(
            torch_weight(name), dtype=dtype, device=self.device, layout=self.model_config["MLP_W_LAYOUT_TILE"],
            memory_config=self.model_config["MLP_WEIGHTS_MEMCFG"], cache_file_name=cache_name(name))
        self.w1 = as_tensor("w1")
        self.w2 = as_tensor("w2")
        self.w3 = as_tensor("w3")

    def forward(self, x):
        w1_out = ttnn.linear(x, self.w1, activation="silu", core_grid=self.args.max_grid_size, use_1d_systolic_array=True,
                             memory_config=self.model_config["FF1_OUTPUT_MEMCFG"],
                             compute_kernel_config=self.args.get_compute_kernel_config())
        w3_out = ttnn.linear(x, self.w3, core_grid=self.args.max_grid_size, use_1d_systolic_array=True,
                             memory_config=self.model_config["FF3_OUTPUT_MEMCFG"],
                             compute_kernel_config=self.args.get_compute_kernel_config())
        w2_in = ttnn.mul(w1_out, w3_out, memory_config=self.model_config["FF3_OUTPUT_MEMCFG"])
        w2_out = ttnn.linear(w2_in, self.w2, core_grid=self.args.max_grid_size, use_1d_systolic_array=True,
                             memory_config=self.model_config["FF2_OUTPUT_MEMCFG"],
                             compute_kernel_config=self.args.get_compute_kernel_config())
        return w2_out
