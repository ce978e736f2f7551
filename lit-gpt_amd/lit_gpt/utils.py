"""Small helpers on the decode path (subset of /root/reference/lit_gpt/utils.py used by generate/*)."""

from __future__ import annotations

import sys
from pathlib import Path


def find_multiple(n: int, k: int) -> int:
    """Smallest multiple of ``k`` that is >= ``n`` (reference lit_gpt/utils.py:74-78)."""
    assert k > 0
    if n % k == 0:
        return n
    return n + k - (n % k)


def check_valid_checkpoint_dir(checkpoint_dir: Path) -> None:
    """Same required files as the reference (lit_gpt/utils.py:93-124); exits with status 1 otherwise."""
    checkpoint_dir = Path(checkpoint_dir)
    files = {
        "lit_model.pth": (checkpoint_dir / "lit_model.pth").is_file(),
        "lit_config.json": (checkpoint_dir / "lit_config.json").is_file(),
        "tokenizer.json OR tokenizer.model": (checkpoint_dir / "tokenizer.json").is_file()
        or (checkpoint_dir / "tokenizer.model").is_file(),
        "tokenizer_config.json": (checkpoint_dir / "tokenizer_config.json").is_file(),
    }
    if checkpoint_dir.is_dir() and all(files.values()):
        return
    problem = (f" is missing the files: {[f for f, ok in files.items() if not ok]!r}" if checkpoint_dir.is_dir()
               else " is not a checkpoint directory")
    print(f"--checkpoint_dir {str(checkpoint_dir.absolute())!r}{problem}.", file=sys.stderr)
    raise SystemExit(1)


def get_default_supported_precision(training: bool) -> str:
    """bf16 on MI355X (reference lit_gpt/utils.py:334-347 picks bf16 when the device supports it)."""
    return "bf16-mixed" if training else "bf16-true"


def read_safetensors(path) -> dict:
    """{name: tensor} of a .safetensors file: an 8-byte little-endian header length, that many bytes of JSON
    (name -> dtype, shape, data_offsets), then the raw little-endian data. Nothing in the file is executed."""
    import json
    import struct

    import numpy as np
    import torch

    kinds = {"BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2), "F32": (torch.float32, 4),
             "F64": (torch.float64, 8), "I32": (torch.int32, 4), "I64": (torch.int64, 8), "U8": (torch.uint8, 1),
             "I8": (torch.int8, 1), "I16": (torch.int16, 2), "BOOL": (torch.bool, 1)}
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    data = np.memmap(path, dtype=np.uint8, mode="r", offset=8 + n)
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        dtype, size = kinds[meta["dtype"]]
        lo, hi = meta["data_offsets"]
        count = 1
        for s in meta["shape"]:
            count *= int(s)
        if hi - lo != count * size:
            raise ValueError(f"{path}: tensor {name!r} has {hi - lo} bytes for shape {meta['shape']}")
        raw = torch.from_numpy(np.array(data[lo:hi]))  # a private copy: the map is read-only
        out[name] = raw.view(dtype).reshape(meta["shape"]) if count else torch.empty(meta["shape"], dtype=dtype)
    return out
