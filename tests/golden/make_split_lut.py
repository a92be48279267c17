"""Regenerate tests/golden/split_lut.json from the reference's host look-up table.

Reads src/base_conv_launchers.h of the reference AS TEXT (it is never compiled
or imported) and writes, for each (kD, kH, kW) key of `splitControl`
(src/base_conv_launchers.h:58-388), the six integer arrays D_s/D_e/H_s/H_e/W_s/W_e.
Only runs where /root/reference exists; the JSON it wrote is the committed fixture.

    python tests/golden/make_split_lut.py
"""
import json
import os
import re
import sys

SRC = "/root/reference/src/base_conv_launchers.h"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "split_lut.json")


def main():
    text = open(SRC).read()
    body = text[text.index("static void splitControl"):]
    key_re = re.compile(r"D == (\d+) && H == (\d+) && W == (\d+)\)\s*\{(.*?)tensorCopy", re.S)
    arr_re = re.compile(r"int (\w+)\[\] = \{([^}]*)\}")
    lut = {}
    for kd, kh, kw, blk in key_re.findall(body):
        arrays = {name: [int(v) for v in vals.split(",") if v.strip()]
                  for name, vals in arr_re.findall(blk)}
        assert set(arrays) == {"D_s", "D_e", "H_s", "H_e", "W_s", "W_e"}, arrays.keys()
        lut["%sx%sx%s" % (kd, kh, kw)] = arrays
    json.dump(lut, open(OUT, "w"), indent=0, sort_keys=True)
    print("wrote %d keys to %s" % (len(lut), OUT))


if __name__ == "__main__":
    sys.exit(main())
