#!/usr/bin/env python3
"""Regenerate include/pf_iq2_codes.h from the reference's IQ2_XXS grid table.

Runs only where /root/reference is mounted.  The output is data: 256 16-bit
words, one 2-bit level index per grid position (0 -> 8, 1 -> 25, 2 -> 43).
tests/test_oracle_packed.py re-expands the words and checks the SHA-256 the
reference records for its 2048-byte table (src/qwen4_iq2_grid.inc:4).
"""
import hashlib
import re
import sys
from pathlib import Path

SOURCE = Path("/root/reference/src/qwen4_iq2_grid.inc")
DIGEST = "05826b5d3e472a3a78f196be62ac78acf81df0f909626e12ab9fa2a5d490dd54"
LEVEL = {8: 0, 25: 1, 43: 2}


def main():
    text = SOURCE.read_text()
    body = text[text.index("*/") + 2:]
    words = [int(w, 16) for w in re.findall(r"0x[0-9a-f]+", body)]
    raw = b"".join(w.to_bytes(8, "little") for w in words)
    if len(words) != 256 or hashlib.sha256(raw).hexdigest() != DIGEST:
        sys.exit("unexpected grid table")
    codes = []
    for w in words:
        code = 0
        for j in range(8):
            code |= LEVEL[(w >> (8 * j)) & 255] << (2 * j)
        codes.append(code)
    for i in range(0, 256, 8):
        print("    " + ", ".join("0x%04x" % c for c in codes[i:i + 8]) + ",")


if __name__ == "__main__":
    main()
