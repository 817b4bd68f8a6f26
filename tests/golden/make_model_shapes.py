"""Writes tests/golden/conv2d_gw8_model_shapes.json.

Reads the shape corpus the reference's tests draw from
(/root/reference/spio/src_tests/Conv2dGw8Params.dat, one
`Conv2dGw8Params(...)` literal per line: 81 layer shapes taken from
EfficientNet / ConvNeXt style models) as text and stores the fields as JSON.
Nothing of the reference is imported or executed.  Run in the build
container only; the JSON is what travels.
"""

import json
import os
import re
import sys

SRC = "/root/reference/spio/src_tests/Conv2dGw8Params.dat"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "conv2d_gw8_model_shapes.json")

LINE = re.compile(
    r"Conv2dGw8Params\(n=(\d+), c=(\d+), h=(\d+), w=(\d+), padding=\((\d+), (\d+)\), "
    r"r=(\d+), s=(\d+), has_bias=(True|False)"
)


def main():
    shapes = []
    with open(SRC, "r", encoding="utf-8") as f:
        for line in f:
            line = line.strip()
            if not line:
                continue
            m = LINE.match(line)
            if m is None:
                sys.exit(f"unparsed line: {line}")
            n, c, h, w, py, px, r, s = (int(v) for v in m.groups()[:8])
            shapes.append(dict(n=n, c=c, h=h, w=w, py=py, px=px, r=r, s=s, has_bias=m.group(9) == "True"))
    with open(OUT, "w", encoding="utf-8") as f:
        json.dump(shapes, f, indent=0)
    print(f"{len(shapes)} shapes -> {OUT}")


if __name__ == "__main__":
    main()
