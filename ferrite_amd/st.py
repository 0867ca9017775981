"""Checkpoint readers for the two formats of the path: a folder of safetensors shards, opened once, tensors read as raw
little-endian bytes. Follows crates/fe-exl3/src/st.rs (shards from model.safetensors.index.json, else
model.safetensors) and crates/fe-fp4/src/st.rs (every *.safetensors of the folder, hf_quant_config.json for the
quantization algorithm of a layer). The header of a shard is 8 bytes of length and that much JSON; nothing else of
the file is interpreted, and nothing in it is executed."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import numpy as np

from .exl3 import Exl3Tensor
from .fp4 import HostLinear, TILE

MUL1 = 0x83DCD12D  # crates/fe-exl3/src/format.rs:14


@dataclass
class TensorInfo:
    dtype: str
    shape: list
    file: int
    offset: int
    nbytes: int


class Checkpoint:
    def __init__(self, folder: str):
        self.dir = folder
        idx = os.path.join(folder, "model.safetensors.index.json")
        if os.path.exists(idx):  # fe-exl3 st.rs:33-46
            with open(idx) as f:
                names = sorted(set(json.load(f)["weight_map"].values()))
        else:  # fe-fp4 st.rs:31-37 (which covers fe-exl3's single model.safetensors)
            names = sorted(p for p in os.listdir(folder) if p.endswith(".safetensors"))
        if not names:
            raise FileNotFoundError(f"{folder}: no safetensors shards")
        self.paths, self.tensors = [], {}
        for fi, name in enumerate(names):
            path = os.path.join(folder, name)
            with open(path, "rb") as f:
                hlen = int.from_bytes(f.read(8), "little")
                header = json.loads(f.read(hlen))
            for key, t in header.items():
                if key == "__metadata__":
                    continue
                a, b = t["data_offsets"]
                self.tensors[key] = TensorInfo(t.get("dtype", ""), list(t["shape"]), fi, 8 + hlen + a, b - a)
            self.paths.append(path)
        self.quant = {}
        try:  # fe-fp4 st.rs:64-68
            with open(os.path.join(folder, "hf_quant_config.json")) as f:
                self.quant = json.load(f)["quantization"]["quantized_layers"]
        except (OSError, KeyError, ValueError):
            pass

    def info(self, name: str) -> TensorInfo:
        if name not in self.tensors:
            raise KeyError(f"tensor {name} not in checkpoint {self.dir}")
        return self.tensors[name]

    def has(self, name: str) -> bool:
        return name in self.tensors

    def read(self, name: str, dtype=np.uint8) -> np.ndarray:
        t = self.info(name)
        if t.nbytes % np.dtype(dtype).itemsize:
            raise ValueError(f"{name}: {t.nbytes} bytes as {np.dtype(dtype).name}")
        with open(self.paths[t.file], "rb") as f:
            f.seek(t.offset)
            data = f.read(t.nbytes)
        if len(data) != t.nbytes:
            raise IOError(f"reading {name} from {self.dir}: the model folder is incomplete or damaged")
        return np.frombuffer(data, dtype=np.dtype(dtype).newbyteorder("<")).astype(dtype, copy=True)

    def scalar(self, name: str) -> float:  # fe-fp4 st.rs:91-98
        t = self.info(name)
        if t.dtype != "F32" or t.nbytes != 4:
            raise ValueError(f"{name}: expected scalar F32, got {t.dtype} {t.shape}")
        return float(self.read(name, np.float32)[0])

    def algo(self, layer: str):  # fe-fp4 st.rs:100-110
        a = self.quant.get(layer, {}).get("quant_algo") if isinstance(self.quant.get(layer), dict) else None
        if a:
            return a
        t = self.tensors.get(f"{layer}.weight")
        if t is None:
            return None
        if t.dtype == "U8" and self.has(f"{layer}.weight_scale_2"):
            return "NVFP4"
        if t.dtype == "F8_E4M3":
            return "FP8"
        return None


def load_exl3(ck: Checkpoint, base: str) -> Exl3Tensor:
    """`base`.trellis / .suh / .svh / .mul1 -> Exl3Tensor; the bit width comes from the trellis shape
    (crates/fe-exl3/src/format.rs:34-57)."""
    tn = f"{base}.trellis"
    info = ck.info(tn)
    if len(info.shape) != 3 or info.shape[2] % 16:
        raise ValueError(f"{tn}: shape {info.shape} (half-integer bit widths unsupported)")
    kt, nt, w = info.shape
    bits = w // 16
    if not 1 <= bits <= 8:
        raise ValueError(f"{tn}: {bits} bits")
    mul = ck.read(f"{base}.mul1", np.uint32)
    if mul.size == 0 or int(mul[0]) != MUL1:
        raise ValueError(f"{base}: codebook is not mul1 ({mul.tolist()})")
    trellis = ck.read(tn, np.uint32)
    suh, svh = ck.read(f"{base}.suh", np.uint16), ck.read(f"{base}.svh", np.uint16)
    k, n = kt * 16, nt * 16
    if suh.size != k or svh.size != n:
        raise ValueError(f"{base}: suh {suh.size} svh {svh.size} for {k}x{n}")
    return Exl3Tensor(base, k, n, bits, trellis, suh, svh)


@dataclass
class Slice:
    """Rows (output features, 128-aligned ranges) and the K range (128-aligned) of one part (lib.rs:245-262)."""
    rows: list
    k: tuple


def select(src: np.ndarray, row_len: int, keep, c0: int, c1: int) -> np.ndarray:
    """Rows `keep` (ranges) and bytes c0..c1 of each, from a row-major byte matrix (lib.rs:420-423 `select`)."""
    m = src.reshape(-1, row_len)
    return np.ascontiguousarray(np.concatenate([m[a:b, c0:c1] for a, b in keep])).reshape(-1)


def load_nvfp4(ck: Checkpoint, parts, slices=None) -> HostLinear:
    """Read and fuse `parts` (layer names without `.weight`) along N, one Slice of each under tensor parallelism
    (crates/fe-fp4/src/lib.rs:305-384, NVFP4 only)."""
    if not parts:
        raise ValueError("no parts")
    if slices is not None and len(slices) != len(parts):
        raise ValueError(f"{parts[0]}: {len(parts)} parts, slices for {len(slices)}")
    fused = []
    for i, p in enumerate(parts):
        algo = ck.algo(p)
        if algo != "NVFP4":
            raise ValueError(f"{p}: not NVFP4 ({algo})")
        t = ck.info(f"{p}.weight")
        fpn, fpk = t.shape[0], t.shape[1] * 2
        codes, sf = ck.read(f"{p}.weight"), ck.read(f"{p}.weight_scale")
        if codes.size != fpn * fpk // 2 or sf.size != fpn * fpk // 16:
            raise ValueError(f"{p}: weight bytes")
        pn, pk = fpn, fpk
        if slices is not None:
            sl = slices[i]
            ok = all(a < b <= fpn and a % TILE == 0 and b % TILE == 0 for a, b in sl.rows)
            ok = ok and sl.k[0] < sl.k[1] <= fpk and sl.k[0] % 128 == 0 and sl.k[1] % 128 == 0
            if not ok:
                raise ValueError(f"{p}: slice {sl} of {fpn}x{fpk}")
            codes = select(codes, fpk // 2, sl.rows, sl.k[0] // 2, sl.k[1] // 2)
            sf = select(sf, fpk // 16, sl.rows, sl.k[0] // 16, sl.k[1] // 16)
            pn, pk = sum(b - a for a, b in sl.rows), sl.k[1] - sl.k[0]
        fused.append((p, codes.reshape(pn, pk // 2), sf.reshape(pn, pk // 16), ck.scalar(f"{p}.weight_scale_2"),
                      ck.scalar(f"{p}.input_scale")))
    return HostLinear.fuse(fused)
