"""Random weights from a configuration and a seed, as a model folder or in memory.

One seeded generator draws every tensor in the order the architecture lists them:
matrices and biases N(0, std), gains 1 + N(0, gain_std), logarithms of rates N(0, 0.5), fractions sigmoid(N(0, 1)), depth weights N(0, 0.15) with 1 added to the last, mixing matrices I + N(0, 0.2), tables
of experts as rows of distinct expert numbers.  Values are drawn in fp32 and rounded
to the storage dtype, so a bfloat16 folder read back in float32 holds the same numbers.
"""

import json
import os

import torch


def random_checkpoint(arch, config, seed: int, dtype=torch.bfloat16, device="cpu", std: float = 0.02,
                      gain_std: float = 0.1) -> dict:  # fmt: skip
    """{checkpoint name: tensor} on `device`, drawn tensor by tensor."""
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = {}
    for name, (shape, role) in arch.checkpoint_shapes(config).items():
        if role.startswith("expert_table:"):  # every row names distinct experts
            experts = int(role.split(":")[1])
            keys = torch.rand((shape[0], experts), generator=gen, device=device)
            out[name] = keys.argsort(dim=1)[:, : shape[1]].to(torch.int32).contiguous()
            continue
        t = torch.randn(tuple(shape), generator=gen, device=device, dtype=torch.float32)
        if role == "vector":
            t = t.mul_(gain_std).add_(1.0)
        elif role == "log_rate":
            t = t.mul_(0.5)
        elif role == "fraction":  # between 0 and 1
            t = torch.sigmoid(t)
        elif role == "depth_weights":  # mostly the last entry, a share of the others
            t = t.mul_(0.15)
            t[-1] += 1.0
        elif role == "near_identity":  # a square matrix that mixes: the identity and a fifth of it in noise
            t = t.mul_(0.2).add_(torch.eye(shape[0], device=device))
        else:
            t = t.mul_(std)
        out[name] = t.to(dtype)
    return out


def write_random_model(path: str, config, seed: int, dtype=torch.bfloat16, std: float = 0.02,
                       gain_std: float = 0.1) -> str:  # fmt: skip
    """Write `path/config.json` and `path/model.safetensors` for a typed configuration."""
    from safetensors.torch import save_file

    from atomserve_amd.config.registry import architecture_for

    raw = config.to_dict()
    raw["torch_dtype"] = str(dtype).replace("torch.", "")  # what the file holds
    arch = architecture_for(raw)
    os.makedirs(path, exist_ok=True)
    tensors = random_checkpoint(arch, config, seed, dtype=dtype, std=std, gain_std=gain_std)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    return path
