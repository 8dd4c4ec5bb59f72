"""Byte-size strings as msccl-tools' plan registry accepts them ('512B', '1MB', '32MiB'): decimal
multiples for KB/MB/GB/TB, binary for KiB/MiB/GiB/TiB, as the humanfriendly package it uses does."""
import math
import re

_UNITS = {"": 1, "b": 1, "byte": 1, "bytes": 1,
          "kb": 10 ** 3, "mb": 10 ** 6, "gb": 10 ** 9, "tb": 10 ** 12, "k": 10 ** 3, "m": 10 ** 6, "g": 10 ** 9, "t": 10 ** 12,
          "kib": 2 ** 10, "mib": 2 ** 20, "gib": 2 ** 30, "tib": 2 ** 40}


def parse_size(text):
    if isinstance(text, (int, float)):
        return int(text)
    m = re.fullmatch(r"\s*([0-9]*\.?[0-9]+)\s*([A-Za-z]*)\s*", str(text))
    if not m or m.group(2).lower() not in _UNITS:
        raise ValueError(f"Failed to parse size! (input {text!r})")
    return int(float(m.group(1)) * _UNITS[m.group(2).lower()])


def format_size(num_bytes):
    if num_bytes == math.inf:
        return "infinity"
    for unit, name in ((10 ** 12, "TB"), (10 ** 9, "GB"), (10 ** 6, "MB"), (10 ** 3, "KB")):
        if num_bytes >= unit:
            value = f"{num_bytes / unit:.2f}".rstrip("0").rstrip(".")
            return f"{value} {name}"
    return f"{int(num_bytes)} byte" + ("" if num_bytes == 1 else "s")
