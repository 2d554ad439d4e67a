#!/usr/bin/env python3
"""Writes PackingTable.inc from the NVCV_PACKING_* enumerator names in include/nvcv/DataLayout.h.

A packing name spells its own layout: fields in storage order, each a channel (X/Y/Z/W + bits) or padding
(b + bits); "_" separates machine words, "__" pixel groups. From that the table row follows:
  fields[4]   widths of the first four fields, padding included (NVCVPackingParams::bits)
  bits[4]     widths of the channels in X, Y, Z, W order (what nvcvPackingGetBitsPerComponent reports)
  order       MSB when fields are separate words ("_") or padding trails the channels, else LSB
  swizzle     for padded packings, the field index (as a channel letter) of every channel, else 0000
  alignment   bytes of one word when the words are equal-sized, else of the whole pixel, as a power of two
(the reference's table: src/nvcv/src/priv/DataLayout.cpp:70-330; its tests: tests/nvcv_types/system/TestDataLayout.cpp:202-420).

usage: python make_packing_table.py   (run from anywhere; rewrites the .inc next to this file)"""
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.normpath(os.path.join(HERE, "..", "..", ".."))


def next_pow2(v):
    p = 1
    while p < v:
        p *= 2
    return p if v > 0 else 0


def row(name):
    body = name[len("NVCV_PACKING_"):]
    words = [w for w in body.split("_") if w]
    fields = []  # (letter or 'b', bits, word index)
    for wi, w in enumerate(words):
        for m in re.finditer(r"([XYZWb])(\d+)", w):
            fields.append((m.group(1), int(m.group(2)), wi))
    letters = [f[0] for f in fields]
    total = sum(f[1] for f in fields)
    padded = "b" in letters
    paired = "__" in body  # 4:2:2 pixel pairs: X8_Y8__X8_Z8
    chan_bits = {}
    for l, b, _ in fields:
        if l != "b":
            chan_bits.setdefault(l, b)
    bits = [chan_bits.get(l, 0) for l in "XYZW"]
    if paired:
        bits = [f[1] for f in fields]  # four stored components
    nwords = len(words)
    if paired:
        order, swz, align = "MSB", "".join(letters), 1
    elif padded:
        first_pad = letters[0] == "b"
        order = "LSB" if (first_pad or (nwords == 1 and letters[-1] != "b")) else "MSB"
        # position (as a letter) of each channel among the fields
        pos = ["XYZW"[i] for i, l in enumerate(letters) if l != "b"]
        swz = "".join(pos).ljust(4, "0")
        word_bits = [sum(f[1] for f in fields if f[2] == wi) for wi in range(nwords)]
        align = next_pow2(word_bits[0] // 8) if len(set(word_bits)) == 1 else next_pow2(max(word_bits) // 8)
        if nwords == 1:
            align = next_pow2(total // 8)
    elif nwords > 1:
        order, swz = "MSB", "0000"
        same = len({f[1] for f in fields}) == 1
        align = next_pow2(fields[0][1] // 8 if same else total // 8)
    else:
        order, swz = "LSB", "0000"
        align = next_pow2(total // 8)
    fw = [f[1] for f in fields][:4] + [0] * (4 - len(fields))
    return '    {%s, "%s", NVCV_ORDER_%s, %d, NVCV_SWIZZLE_%s, {%s}, {%s}},' % (
        name, name, order, align, swz, ", ".join(map(str, fw)), ", ".join(map(str, bits)))


def main():
    text = open(os.path.join(ROOT, "include", "nvcv", "DataLayout.h")).read()
    enum = text[text.index("NVCV_PACKING_0 = 0"):text.index("} NVCVPacking;")]
    names = [n for n in re.findall(r"\b(NVCV_PACKING_\w+)\b\s*(?:=|,)", enum) if n not in ("NVCV_PACKING_0", "NVCV_PACKING_LIMIT32")]
    out = ["// {packing, name, byte order, alignment, swizzle as stored, widths of the stored fields (padding included),",
           "//  bits of the channels X Y Z W}; written by make_packing_table.py from the enumerator names in nvcv/DataLayout.h"]
    out += [row(n) for n in names]
    open(os.path.join(HERE, "PackingTable.inc"), "w").write("\n".join(out) + "\n")
    print(len(names), "packings")


if __name__ == "__main__":
    main()
