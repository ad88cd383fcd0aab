"""Writes tests/golden/f16_shortest_decimals_sample.txt: every 16th line of the reference's table of all
65536 f16 bit patterns with their shortest decimal strings (nx/test/fixtures/f16_table.txt, the data
file of nx/test/nx/ryu_test.exs), plus the neighbourhoods where an f16 codec goes wrong first: the
subnormals next to zero, the step to the normals, one, the largest finite values, the infinities and
the first NaNs of either sign.  Data only; run once where the reference tree is present:
    python tests/golden/make_f16_sample.py /root/reference/nx/test/fixtures/f16_table.txt
"""
import os
import sys

src = sys.argv[1]
lines = open(src).read().split("\n")
lines = [l for l in lines if l]
keep = set(range(0, 65536, 16))
for centre in (0x0000, 0x0400, 0x3C00, 0x7BFF, 0x7C00, 0x8000, 0x8400, 0xBC00, 0xFBFF, 0xFC00):
    keep.update(i for i in range(centre - 8, centre + 9) if 0 <= i < 65536)
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "f16_shortest_decimals_sample.txt")
with open(out, "w") as f:
    for i in sorted(keep):
        assert int(lines[i].split(":")[0], 16) == i
        f.write(lines[i] + "\n")
print(len(keep), "lines ->", out)
