"""Writes the small golden fixtures under tests/golden/ from data files the
reference's own tests hold.  Run in the build container (needs /root/reference):

    python tests/golden/make_fixtures.py

basic_chain.json <- tests/basic.testdata: the `.matrix` layout is three
little-endian int32 (numrow, numcol, transpose) followed by the column-major
float32 payload (cpp/core.hpp:518-525).
"""
import json
import struct
from pathlib import Path

REF = Path("/root/reference")
OUT = Path(__file__).resolve().parent


def main():
    raw = (REF / "tests" / "basic.testdata").read_bytes()
    numrow, numcol, transpose = struct.unpack("<3i", raw[:12])
    data = struct.unpack(f"<{numrow * numcol}f", raw[12:12 + 4 * numrow * numcol])
    (OUT / "basic_chain.json").write_text(json.dumps(
        {"source": "tests/basic.testdata", "numrow": numrow, "numcol": numcol, "transpose": transpose,
         "data": [float.hex(x) for x in data], "data_decimal": list(data)}, indent=1))


if __name__ == "__main__":
    main()
