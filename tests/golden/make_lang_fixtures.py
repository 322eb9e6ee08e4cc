"""Copies the front-end golden dumps held by the reference's own tests
(tc/lang/test_expected/*.expected, compared byte-for-byte by test/test_lang.cc:88-110) into
tests/golden/lang/, dropping the '#' licence banner the files carry.  Data only: no reference
code is imported or executed.  Run once in a container that mounts the reference:

    python tests/golden/make_lang_fixtures.py /root/reference
"""
import os
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
src = os.path.join(ref, "tc", "lang", "test_expected")
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lang")
os.makedirs(dst, exist_ok=True)
for name in sorted(os.listdir(src)):
    if not name.endswith(".expected"):
        continue
    lines = open(os.path.join(src, name)).read().split("\n")
    i = 0
    while i < len(lines) and lines[i].startswith("#"):
        i += 1
    with open(os.path.join(dst, name), "w") as f:
        f.write("\n".join(lines[i:]))
    print("wrote", name)
