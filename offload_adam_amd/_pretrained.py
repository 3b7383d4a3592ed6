"""Refill fp32 masters of quantised parameters from a bf16/fp16 safetensors
checkpoint (``{Adam,OffloadAdam}.load_master_from_pretrained``).

Checkpoint IO on the host, no kernels: counterpart of the reference's
``_pretrained`` module (src/offload_adam/_pretrained.py).  Tensors are read one
at a time so host memory stays at about one tensor.
"""

import json
from pathlib import Path
from typing import List, Union

import torch

from .qweight.base import QWeightBase


def _files_in(directory: Path) -> List[Path]:
    index = directory / "model.safetensors.index.json"
    if index.exists():
        shard_names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
        return [directory / name for name in shard_names]
    single = directory / "model.safetensors"
    if single.exists():
        return [single]
    loose = sorted(directory.glob("*.safetensors"))
    if not loose:
        raise FileNotFoundError(
            f"No safetensors files under {directory} (looked for model.safetensors, "
            f"model.safetensors.index.json, or any *.safetensors)."
        )
    return loose


def resolve_safetensors_paths(pretrained_name_or_path: Union[str, Path]) -> List[Path]:
    """A file, a (possibly sharded) directory, or a HuggingFace Hub repo id ->
    local safetensors files.  The Hub needs ``huggingface_hub`` and a network."""
    local = Path(pretrained_name_or_path)
    if local.is_file():
        return [local]
    if local.is_dir():
        return _files_in(local)
    try:
        from huggingface_hub import snapshot_download
    except ImportError as exc:
        raise ImportError(
            f"'{pretrained_name_or_path}' is not a local file or directory and "
            "`huggingface_hub` is not installed. Install it or pass a local path."
        ) from exc
    fetched = snapshot_download(
        repo_id=str(pretrained_name_or_path),
        allow_patterns=["*.safetensors", "*.safetensors.index.json"],
    )
    return _files_in(Path(fetched))


@torch.no_grad()
def stream_master_from_pretrained(optim, pretrained_name_or_path, model, *, strict: bool):
    """Copy each checkpoint tensor that names a quantised parameter into that
    parameter's ``master_params`` (widening to fp32 is lossless) and mark it
    ``master_filled``.  Returns the sorted names that no file provided."""
    from safetensors import safe_open

    trainable = {n: p for n, p in model.named_parameters() if p.requires_grad}
    wanted = {n for n, p in trainable.items() if isinstance(p.data, QWeightBase)}
    lazy_init = getattr(optim, "_init_state_if_empty", None)  # Adam creates state lazily
    done = set()
    for path in resolve_safetensors_paths(pretrained_name_or_path):
        with safe_open(str(path), framework="pt", device="cpu") as reader:
            for key in wanted.intersection(reader.keys()):
                param = trainable[key]
                state = optim.state[param]
                if lazy_init is not None:
                    lazy_init(param, state)
                if "master_params" not in state:
                    continue
                optim._copy_master(param, reader.get_tensor(key))
                if "master_filled" in state:
                    state["master_filled"] = True
                done.add(key)
    missing = sorted(wanted - done)
    if strict and missing:
        raise ValueError(
            f"load_master_from_pretrained(strict=True): {len(missing)} quant param(s) "
            f"have no matching key in the checkpoint: {missing}"
        )
    return missing
