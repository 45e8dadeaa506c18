"""HF safetensors checkpoint -> AXM1 file.

Mirror of the reference's converter (axono/python/examples/vlm/qwen3vl/convert.py:32-64): tensor names
are kept as they are (`model.visual.*` / `model.language_model.*` already are the model's flat
parameter names), every tensor is widened to fp32 unless `--dtype` says otherwise,
`patch_embed.proj.weight` is flattened to (out, 3*patch*patch*...), the result goes to
`<model_dir>/model.axm` by default, and the index carries the same `meta` keys.

The safetensors container is read directly (8-byte little-endian header length, a JSON header with
dtype / shape / data_offsets per tensor, then the raw bytes): tensors are memory-mapped and converted
one at a time, bf16 included (numpy has no bf16: the 16 bits become the upper half of an fp32), so the
conversion needs neither torch nor room for the whole checkpoint.  A sharded checkpoint
(`model.safetensors.index.json`) is read shard by shard; the reference reads the single file only.

    python -m axono_amd.format.convert --model /path/to/qwen3vl-2b [--out model.axm] [--dtype float16]
"""
from __future__ import annotations

import argparse
import json
import os
import struct
import sys
import time

import numpy as np

from .axm import write_axm

_ST_DTYPES = {"F64": np.float64, "F32": np.float32, "F16": np.float16, "I64": np.int64, "I32": np.int32,
              "I16": np.int16, "I8": np.int8, "U8": np.uint8, "BOOL": np.bool_}


def read_safetensors_index(path: str):
    """{name: (dtype string, shape, begin, end)} and the byte offset where tensor data starts."""
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: not a safetensors file (short header)")
        (n,) = struct.unpack("<Q", head)
        if n <= 0 or n > os.path.getsize(path) - 8:
            raise ValueError(f"{path}: not a safetensors file (header length {n})")
        header = json.loads(f.read(n).decode("utf-8"))
    header.pop("__metadata__", None)
    return {k: (v["dtype"], tuple(v["shape"]), *v["data_offsets"]) for k, v in header.items()}, 8 + n


def _tensor(path: str, base: int, dtype: str, shape, begin: int, end: int) -> np.ndarray:
    """One tensor of a safetensors file as a numpy array (memory-mapped where no conversion is needed)."""
    if dtype == "BF16":
        count = (end - begin) // 2
        bits = np.memmap(path, dtype="<u2", mode="r", offset=base + begin, shape=(count,)) if count else \
            np.zeros(0, "<u2")
        return (bits.astype(np.uint32) << 16).view(np.float32).reshape(shape)
    if dtype not in _ST_DTYPES:
        raise ValueError(f"{path}: dtype {dtype} is not supported")
    dt = np.dtype(_ST_DTYPES[dtype])
    count = (end - begin) // dt.itemsize
    if count == 0:
        return np.zeros(shape, dt)
    return np.memmap(path, dtype=dt.newbyteorder("<"), mode="r", offset=base + begin, shape=(count,)).reshape(shape)


def _shards(model_dir: str):
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.exists(single):
        return [single]
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index, "r", encoding="utf-8") as f:
            files = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(model_dir, name) for name in files]
    raise FileNotFoundError(f"no model.safetensors (or model.safetensors.index.json) in {model_dir}")


def convert(model_dir: str, out_path: str, dtype: str | None = None) -> dict:
    """Converts the checkpoint in `model_dir`; returns {"n_tensors", "size_gb", "t_read", "t_write"}
    like the reference (reading and writing are interleaved here, so t_read is the indexing time)."""
    t0 = time.perf_counter()
    specs = []
    for shard in _shards(model_dir):
        index, base = read_safetensors_index(shard)
        for name, (dt, shape, begin, end) in index.items():
            if name.endswith("patch_embed.proj.weight"):
                out_shape = (shape[0], int(np.prod(shape[1:], dtype=np.int64)))
            else:
                out_shape = shape
            # everything is widened to fp32 (the dtype the operators compute in) unless a storage dtype
            # is given - integer tensors too, as the reference's `.float()` does
            out_dt = np.dtype(dtype) if dtype else np.dtype(np.float32)
            specs.append((name, out_dt, out_shape,
                          lambda s=shard, b=base, d=dt, sh=shape, o=out_shape, bg=begin, en=end:
                          _tensor(s, b, d, sh, bg, en).reshape(o)))
    t_read = time.perf_counter() - t0
    meta = {"source": "hf-safetensors", "model_dir": os.path.basename(os.path.normpath(model_dir)),
            "converted_at": time.strftime("%Y-%m-%dT%H:%M:%S"), "dtype": dtype or "keep"}
    t1 = time.perf_counter()
    write_axm(specs, out_path, meta)
    t_write = time.perf_counter() - t1
    return {"n_tensors": len(specs), "size_gb": os.path.getsize(out_path) / 1e9, "t_read": t_read, "t_write": t_write}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="HF safetensors -> AXM1")
    ap.add_argument("--model", required=True, help="HF model directory")
    ap.add_argument("--out", default=None, help="output .axm path (default <model>/model.axm)")
    ap.add_argument("--dtype", default=None, choices=["float32", "float16"],
                    help="one storage dtype for every tensor (default: float32)")
    args = ap.parse_args(argv)
    out = args.out or os.path.join(args.model, "model.axm")
    st = convert(args.model, out, args.dtype)
    print(f"converted: {out}")
    print(f"  {st['n_tensors']} tensors, {st['size_gb']:.2f} GB, index {st['t_read']:.1f}s + convert/write {st['t_write']:.1f}s")
    return 0


if __name__ == "__main__":
    sys.exit(main())
