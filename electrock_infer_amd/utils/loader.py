"""Checkpoint loading for the modules of this package, with the reference's dispatch rules
(electrock_infer/utils/loader.py:14-49): every tensor of every ``*.safetensors`` file under ``path`` goes
to the ``weight_loader`` of the parameter it belongs to --

* names that contain a key of ``model.packed_modules_mapping`` are renamed and loaded with a shard id
  (``q_proj`` -> ``qkv_proj`` ...; this package has no such module, a model that embeds ours may),
* expert tensors ``...experts.<e>.w1|w2|w3.weight`` (tensor names as in utils/mixtral_info.txt:17-42) go to the
  stacked ``...experts.w13_weight`` / ``w2_weight`` through ``FusedMoE.weight_loader(param, tensor, shard, e)``,
* everything else is copied by the parameter's own ``weight_loader`` or ``default_weight_loader``.

``strict=False`` skips tensors the model has no parameter for (a model made of the MoE block alone against a
full checkpoint); the reference raises there, and so does ``strict=True``.
"""
import os
from glob import glob
from typing import Dict, List, Tuple

import torch
from torch import nn
from safetensors import safe_open

# expert tensors -> (stacked parameter, shard id): models/mixtral.py:236-240
EXPERTS_MODULES_MAPPING: Dict[str, Tuple[str, str]] = {
    "w1": ("w13_weight", "w1"),
    "w3": ("w13_weight", "w3"),
    "w2": ("w2_weight", "w2"),
}


def default_weight_loader(param: nn.Parameter, loaded_weight: torch.Tensor):
    param.data.copy_(loaded_weight)


def _find(model: nn.Module, name: str, strict: bool):
    try:
        return model.get_parameter(name)
    except AttributeError:
        if strict:
            raise
        return None


def load_model(model: nn.Module, path: str, rank: int = 0, device: str = "cpu", strict: bool = True) -> List[str]:
    """Load every ``*.safetensors`` file under ``path`` into ``model``; returns the names that were loaded."""
    packed = getattr(model, "packed_modules_mapping", {})
    experts = getattr(model, "experts_modules_mapping", EXPERTS_MODULES_MAPPING)
    loaded: List[str] = []
    for file in sorted(glob(os.path.join(path, "*.safetensors"))):
        with safe_open(file, "pt", device) as f:
            for weight_name in f.keys():
                done = False
                for k in packed:
                    if k in weight_name:
                        v, shard_id = packed[k]
                        param = _find(model, weight_name.replace(k, v), strict)
                        if param is not None:
                            param.weight_loader(param, f.get_tensor(weight_name), shard_id)
                            loaded.append(weight_name)
                        done = True
                        break
                if done:
                    continue
                parts = weight_name.split(".")
                # ['model', 'layers', '0', 'block_sparse_moe', 'experts', '<e>', 'w1', 'weight']
                if len(parts) >= 4 and parts[-1] == "weight" and parts[-2] in experts and parts[-3].isdigit() \
                        and parts[-4] == "experts":
                    v, shard_id = experts[parts[-2]]
                    param = _find(model, ".".join(parts[:-3]) + "." + v, strict)
                    if param is not None:
                        param.weight_loader(param, f.get_tensor(weight_name), shard_id, int(parts[-3]))
                        loaded.append(weight_name)
                    continue
                param = _find(model, weight_name, strict)
                if param is not None:
                    getattr(param, "weight_loader", default_weight_loader)(param, f.get_tensor(weight_name))
                    loaded.append(weight_name)
    return loaded
