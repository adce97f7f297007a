#!/usr/bin/env python3
"""Writes tests/golden/iq_codebook_digests.json: SHA-256 digests and spot entries of the importance-quant codebooks as
the reference spells them out.

The tables are read as TEXT from the reference's Rust sources (nothing of the reference is imported, compiled or run):
    crates/rnb-core/src/quant_codebooks.rs:3    KSIGNS_IQ2XS   [u8; 128]
    crates/rnb-core/src/quant_codebooks.rs:13   IQ2XXS_GRID    [u64; 256]
    crates/rnb-core/src/quant_codebooks.rs:787  IQ2S_GRID      [u64; 1024]
    crates/rnb-core/src/quant_codebooks.rs:1814 IQ3XXS_GRID    [u32; 256]
    crates/rnb-cpu/src/quantize/iq.rs:9         KVALUES_IQ4NL  [i8; 16]
The digest of a table is SHA-256 over its entries as little-endian integers of the declared width, in order.  Run in the
build container (the reference is not present on the GPU box); the JSON it writes is the committed fixture that
tests/test_oracle_pins.py::test_iq_codebooks_equal_the_references_tables_entry_for_entry checks the oracle's and the
product's packed tables against.

    python tests/golden/make_iq_codebook_digests.py [/root/reference]
"""
import hashlib
import json
import os
import re
import sys

WIDTH = {"u8": 1, "i8": 1, "u32": 4, "u64": 8}


def table(text, name):
    m = re.search(r"const\s+" + name + r"\s*:\s*\[(\w+);\s*(\d+)\]\s*=\s*\[(.*?)\];", text, re.S)
    if not m:
        raise SystemExit(f"{name} not found")
    ty, n, body = m.group(1), int(m.group(2)), m.group(3)
    body = re.sub(r"//[^\n]*", "", body)
    vals = [int(tok.replace("_", ""), 0) for tok in re.findall(r"-?(?:0x[0-9a-fA-F_]+|\d[\d_]*)", body)]
    if len(vals) != n:
        raise SystemExit(f"{name}: {len(vals)} entries, declared {n}")
    return ty, vals


def digest(ty, vals):
    w = WIDTH[ty]
    raw = b"".join(int(v).to_bytes(w, "little", signed=ty.startswith("i")) for v in vals)
    return hashlib.sha256(raw).hexdigest()


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    books = open(os.path.join(ref, "crates/rnb-core/src/quant_codebooks.rs")).read()
    iq = open(os.path.join(ref, "crates/rnb-cpu/src/quantize/iq.rs")).read()
    out = {}
    for name, text in (("KSIGNS_IQ2XS", books), ("IQ2XXS_GRID", books), ("IQ2S_GRID", books), ("IQ3XXS_GRID", books),
                       ("KVALUES_IQ4NL", iq)):
        ty, vals = table(text, name)
        spots = sorted({0, 1, len(vals) // 3, len(vals) // 2, len(vals) - 2, len(vals) - 1})
        out[name] = {"type": ty, "entries": len(vals), "sha256": digest(ty, vals), "spot": {str(i): vals[i] for i in spots}}
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "iq_codebook_digests.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", dst)


if __name__ == "__main__":
    main()
