"""Reading and writing the reference's ``.mdlus`` model checkpoints (physicsnemo/core/module.py:446-640, :689-800,
:800-1070): an archive -- zip by default, tar in the legacy format -- holding

  model.pt        ``torch.save`` of the state dict
  args.json       {"__name__": class name, "__module__": defining module, "__args__": constructor arguments}
  metadata.json   {"physicsnemo_version": ..., "mdlus_file_version": ...}

Only the tensors are ever deserialised (``torch.load(weights_only=True)``); nothing in a checkpoint is executed.
"""
from __future__ import annotations

import io
import json
import tarfile
import zipfile

import torch

MDLUS_FILE_VERSION = "0.1.0"
_EXPECTED = ("args.json", "metadata.json", "model.pt")


def read_mdlus(path: str, map_location="cpu"):
    """Returns (args dict, metadata dict, state dict) of a zip- or tar-format ``.mdlus`` file."""
    # the tar check comes first: a tar archive holds model.pt, itself a zip file, which zipfile would recognise
    # (module.py:657-660)
    if tarfile.is_tarfile(path):  # legacy format (module.py:609-633)
        with tarfile.open(path, "r") as tar:
            members = {m.name.lstrip("./"): m for m in tar.getmembers() if m.isfile()}
            for name in _EXPECTED:
                if name not in members:
                    raise IOError(f"File '{name}' not found in checkpoint")
            blobs = {name: tar.extractfile(members[name]).read() for name in _EXPECTED}
    elif zipfile.is_zipfile(path):
        with zipfile.ZipFile(path, "r") as archive:
            names = archive.namelist()
            for name in _EXPECTED:
                if name not in names:
                    raise IOError(f"File '{name}' not found in checkpoint")
            blobs = {name: archive.read(name) for name in _EXPECTED}
    else:
        raise IOError(f"{path} is neither a zip nor a tar archive: not a .mdlus checkpoint")
    args = json.loads(blobs["args.json"])
    metadata = json.loads(blobs["metadata.json"])
    state = torch.load(io.BytesIO(blobs["model.pt"]), map_location=map_location, weights_only=True)
    return args, metadata, state


def write_mdlus(path: str, class_name: str, module_name: str, ctor_args: dict, state_dict: dict) -> None:
    """Writes the default (zip) format the reference writes (module.py:585-606)."""
    if not str(path).endswith(".mdlus"):
        raise ValueError("File name must end with .mdlus extension")
    buf = io.BytesIO()
    torch.save({k: v.detach().cpu() for k, v in state_dict.items()}, buf)
    args = {"__name__": class_name, "__module__": module_name, "__args__": ctor_args}
    metadata = {"physicsnemo_version": "physicsnemo_amd", "mdlus_file_version": MDLUS_FILE_VERSION}
    with zipfile.ZipFile(path, "w", zipfile.ZIP_STORED) as archive:
        archive.writestr("model.pt", buf.getvalue())
        archive.writestr("args.json", json.dumps(args))
        archive.writestr("metadata.json", json.dumps(metadata))
