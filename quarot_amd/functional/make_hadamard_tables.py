"""Build ``hadamard_tables.bin`` from the text of the reference's Hadamard tables.

The eleven +-1 matrices (orders 12, 20, 28, 36, 40, 52, 60, 108, 140, 156, 172; Sloane's
library) are data that weights rotated offline by the reference depend on verbatim
(reference: quarot/functional/hadamard.py:153-4193, identical copy in
fake_quant/hadamard_utils.py).  This script parses that file AS TEXT (nothing is imported or
executed), checks H.H^T = K.I, and writes every matrix bit-packed (row-major, +1 -> bit 1,
numpy.packbits big-endian bit order), concatenated in ascending order of K.

Usage:  python make_hadamard_tables.py /root/reference/quarot/functional/hadamard.py
"""
import hashlib
import pathlib
import re
import sys

import numpy as np

ORDERS = (12, 20, 28, 36, 40, 52, 60, 108, 140, 156, 172)


def parse_tables(text):
    """Return {K: int8 [K, K]} from ``def get_hadK(): return torch.FloatTensor([...])`` bodies."""
    out = {}
    heads = list(re.finditer(r"^def get_had(\d+)\(\):", text, flags=re.M))
    for i, h in enumerate(heads):
        k = int(h.group(1))
        end = heads[i + 1].start() if i + 1 < len(heads) else len(text)
        toks = re.findall(r"[+-]1\b", text[h.end():end])
        if len(toks) != k * k:
            raise ValueError(f"had{k}: {len(toks)} entries, expected {k * k}")
        out[k] = np.array([1 if t[0] == "+" else -1 for t in toks], dtype=np.int8).reshape(k, k)
    return out


def main(src, dst):
    tables = parse_tables(pathlib.Path(src).read_text())
    if tuple(sorted(tables)) != ORDERS:
        raise ValueError(f"orders found: {sorted(tables)}")
    blob = bytearray()
    for k in ORDERS:
        h = tables[k].astype(np.int64)
        if not np.array_equal(h @ h.T, k * np.eye(k, dtype=np.int64)):
            raise ValueError(f"had{k} is not orthogonal")
        bits = np.packbits(h.reshape(-1) > 0)
        print(k, hashlib.sha256(bits.tobytes()).hexdigest()[:16])
        blob += bits.tobytes()
    pathlib.Path(dst).write_bytes(bytes(blob))
    print("wrote", dst, len(blob), "bytes")


if __name__ == "__main__":
    here = pathlib.Path(__file__).resolve().parent
    main(sys.argv[1], here / "hadamard_tables.bin")
