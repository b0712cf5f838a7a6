"""cccc's weight container ("CFG_BIN INI"), writer and pure-Python reader.

Layout as scripts/convert_weights.py:54-83 writes it: 32 bytes "CFG_BIN INI" zero-padded, a
little-endian uint64 with the length of the index text, the index text (ASCII lines
"<key> = <offset>,<length>", offsets relative to the data area), then the data area.  The C++ reader and
writer the product uses are cccc-lite_amd/host/WeightFile.cpp; this module is test infrastructure: it makes
files for tests and reads them back without the native library.
"""
from __future__ import annotations

import struct
from pathlib import Path

import numpy as np

MAGIC = b"CFG_BIN INI"
HEADER_BYTES = 32


class BinWriter:
    def __init__(self):
        self.entries: dict[str, bytes] = {}

    def add(self, key: str, data) -> None:
        self.entries[key] = data.tobytes() if isinstance(data, np.ndarray) else bytes(data)

    def add_float(self, key: str, value: float) -> None:
        self.entries[key] = struct.pack("<f", value)

    def save(self, filename) -> int:
        lines, offset = [], 0
        for key, val in self.entries.items():
            lines.append(f"{key} = {offset},{len(val)}")
            offset += len(val)
        ini = ("\n".join(lines) + "\n").encode("ascii")
        with open(filename, "wb") as f:
            f.write(MAGIC + b"\x00" * (HEADER_BYTES - len(MAGIC)))
            f.write(struct.pack("<Q", len(ini)))
            f.write(ini)
            for val in self.entries.values():
                f.write(val)
        return HEADER_BYTES + 8 + len(ini) + offset


def read_index(filename) -> tuple[dict[str, tuple[int, int]], int]:
    """{key: (offset, length)} and the file offset of the data area."""
    with open(filename, "rb") as f:
        head = f.read(HEADER_BYTES + 8)
        if len(head) < HEADER_BYTES + 8 or not head.startswith(MAGIC):
            raise ValueError("not a CFG_BIN INI file")
        (ini_len,) = struct.unpack("<Q", head[HEADER_BYTES:])
        ini = f.read(ini_len).decode("ascii")
    index = {}
    for line in ini.splitlines():
        line = line.strip()
        if not line or line[0] in "[;#":
            continue
        key, _, rest = line.partition("=")
        off, _, length = rest.partition(",")
        index[key.strip()] = (int(off), int(length))
    return index, HEADER_BYTES + 8 + ini_len


def read_entry(filename, key: str) -> bytes:
    index, base = read_index(filename)
    off, length = index[key]
    with open(filename, "rb") as f:
        f.seek(base + off)
        return f.read(length)


def write_decode_model(filename, model: dict, linear_key: str = "fp8_e5m2", scales: dict | None = None) -> int:
    """Writes a model in the dict layout of the decode oracle (emb, rms_final, lm_head, layers[...]) under the
    converter's names (scripts/convert_weights.py:142-166).  Linears go out as `linear_key` bytes."""
    names = {"rms_attn": "W_rms_attn", "wq": "W_q", "wk": "W_k", "wv": "W_v", "q_norm": "W_qnorm", "k_norm": "W_knorm", "wo": "W_o",
             "rms_ffn": "W_rms_ffn", "w_gate": "W_gate", "w_up": "W_up", "w_down": "W_down"}
    linears = {"wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"}
    w = BinWriter()
    w.add("named_weights", b"1")
    w.add("weight_bf16_W_emb", model["emb"])
    w.add("weight_bf16_W_rms_final", model["rms_final"])
    w.add(f"weight_{linear_key}_W_lm_head", model["lm_head"])
    for i, layer in enumerate(model["layers"]):
        for short, arr in layer.items():
            name = f"{names[short]}_{i}"
            w.add(f"weight_{linear_key if short in linears else 'bf16'}_{name}", arr)
            if scales and name in scales:
                w.add_float(f"scale_{name}", scales[name])
    if scales and "W_lm_head" in scales:
        w.add_float("scale_W_lm_head", scales["W_lm_head"])
    return w.save(Path(filename))
