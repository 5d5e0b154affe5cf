"""CPU restatement (test infrastructure only) of the KV snapshot wire format of one MLA layer:
write_mla_layer / read_mla_layer (src/runtime/glm52/rocm_swap.rs:1090-1138) over the primitive encoders
write_usize / write_bytes (rocm_swap.rs:1145-1153) and CacheReader (rocm_swap.rs:1160-1208).  A record is the
reference's MlaLayerSerde (src/backend/rocm/kv_cache.rs:2067-2083)."""
import struct
from dataclasses import dataclass
from typing import Optional

OWNERSHIP = {"Full": 0, "BlockParity(0)": 1, "BlockParity(1)": 2, "InterleavedPair": 3}


@dataclass
class MlaLayerSerde:
    rows: int
    ownership: str
    latent_cols: int
    rope_cols: int
    latent_group_size: int
    latent: bytes
    latent_scales: Optional[bytes]
    rope: bytes


def _usize(value: int) -> bytes:  # rocm_swap.rs:1145-1148
    return struct.pack("<Q", value)


def _blob(data: bytes) -> bytes:  # rocm_swap.rs:1150-1153
    return _usize(len(data)) + bytes(data)


def write_mla_layer(layer: MlaLayerSerde) -> bytes:  # rocm_swap.rs:1090-1113
    out = _usize(layer.rows) + bytes([OWNERSHIP[layer.ownership]])
    out += _usize(layer.latent_cols) + _usize(layer.rope_cols) + _usize(layer.latent_group_size)
    out += _blob(layer.latent)
    out += b"\x00" if layer.latent_scales is None else b"\x01" + _blob(layer.latent_scales)
    return out + _blob(layer.rope)


class _Reader:  # rocm_swap.rs:1160-1208
    def __init__(self, data: bytes):
        self.data, self.at = bytes(data), 0

    def take(self, n: int) -> bytes:
        if n > len(self.data) - self.at:
            raise ValueError(f"truncated: need {n}, {len(self.data) - self.at} left")
        self.at += n
        return self.data[self.at - n:self.at]

    def usize(self) -> int:
        return struct.unpack("<Q", self.take(8))[0]

    def byte(self) -> int:
        return self.take(1)[0]

    def flag(self) -> bool:
        value = self.byte()
        if value > 1:
            raise ValueError(f"flag={value}")
        return value == 1

    def blob(self) -> bytes:
        return self.take(self.usize())


def read_mla_layer(data: bytes):  # rocm_swap.rs:1123-1139; returns (record, bytes consumed)
    reader = _Reader(data)
    rows = reader.usize()
    code = reader.byte()
    names = {v: k for k, v in OWNERSHIP.items()}
    if code not in names:
        raise ValueError(f"ownership={code}")
    latent_cols, rope_cols, group = reader.usize(), reader.usize(), reader.usize()
    latent = reader.blob()
    scales = reader.blob() if reader.flag() else None
    rope = reader.blob()
    return MlaLayerSerde(rows, names[code], latent_cols, rope_cols, group, latent, scales, rope), reader.at
