#!/usr/bin/env python3
"""Writes image_format_vectors.json: the per-format expectations the reference's own unit test holds
(tests/nvcv_types/system/TestImageFormat.cpp:93-308, the parameter table of ImageFormatTests), restated as data:
for every listed format its colour model, colour spec, chroma subsampling, memory layout, swizzle, alpha type,
plane packings, data kind, chroma samples, bits per channel, plane count, per-plane {bits per pixel, channels, data
type, swizzle} and extra-channel info. Enumerators are kept by name; the test resolves them against this build's
constant table.

usage: python tests/golden/make_image_format_vectors.py [/root/reference]"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
text = open(os.path.join(ref, "tests/nvcv_types/system/TestImageFormat.cpp")).read()
body = text[text.index("INSTANTIATE_TEST_SUITE_P(\n    ExplicitTypes, ImageFormatTests"):text.index("TEST_P(ImageFormatTests, make_image_format)")]
body = re.sub(r"\s+", "", body)
pat = re.compile(r"Params\{(NVCV_IMAGE_FORMAT_\w+),FMT_IMAGE_PARAMS\(([^)]*)\),(\d+),(\d+),(NVCV_CHROMA_LOC_\w+),(NVCV_CHROMA_LOC_\w+),"
                 r"\{([^}]*)\},(\d+),\{((?:\{[^}]*\},?)+)\},\{([^}]*)\}\}")
rows = []
for m in pat.finditer(body):
    model, spec, css, layout, kind, swz, alpha, p0, p1, p2, p3 = m.group(2).split(",")
    planes = [dict(zip(("bpp", "channels", "dataType", "swizzle"), [int(a), int(b), c, d]))
              for a, b, c, d in re.findall(r"\{(\d+),(\d+),(\w+),(\w+)\}", m.group(9))]
    ex = m.group(10).split(",")
    rows.append({"format": m.group(1), "colorModel": model, "colorSpec": spec, "css": css, "memLayout": layout, "dataKind": kind,
                 "swizzle": swz, "alphaType": alpha, "packings": [p0, p1, p2, p3], "samplesHoriz": int(m.group(3)),
                 "samplesVert": int(m.group(4)), "bitsPerChannel": [int(v) for v in m.group(7).split(",")],
                 "planeCount": int(m.group(8)), "planes": planes,
                 "extra": {"numChannels": int(ex[0]), "bitsPerPixel": int(ex[1]), "dataKind": ex[2], "channelType": ex[3]}})
assert body.count("Params{") == len(rows), (body.count("Params{"), len(rows))
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "image_format_vectors.json")
open(out, "w").write("[\n" + ",\n".join(json.dumps(r) for r in rows) + "\n]\n")
print(len(rows), "formats")
