"""Extracts the known answers of the reference's range-inference tests (test/test_inference.cc:70-540:
each test hands a TC definition to Check() together with the expected "mins:" / "extents:" text, the
bounds of every tensor as expressions of the size parameters) into
tests/golden/inference/known_answers.json — definitions and expected texts only, data the reference's
test holds; no reference code is imported or executed.  Run once in a container that mounts the reference:

    python tests/golden/make_inference_fixtures.py /root/reference
"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
text = open(os.path.join(ref, "test", "test_inference.cc")).read()
cases = []
heads = list(re.finditer(r"TEST_F\(InferenceTest, (\w+)\) \{", text))
for i, m in enumerate(heads):
    name = m.group(1)
    body = text[m.end():heads[i + 1].start() if i + 1 < len(heads) else len(text)]
    inline = re.search(r'Check\(\s*R"\((.*?)\)",\s*R"HALIDE\((.*?)\)HALIDE"\)', body, re.S)
    named = re.search(r'R"TC\((.*?)\)TC";.*?Check\(tc, R"HALIDE\((.*?)\)HALIDE"\)', body, re.S)
    hit = inline or named
    if hit and "EXPECT_THROW" not in body:
        cases.append({"name": name, "tc": hit.group(1), "expected": hit.group(2)})
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "inference")
os.makedirs(dst, exist_ok=True)
with open(os.path.join(dst, "known_answers.json"), "w") as f:
    json.dump(cases, f, indent=1)
print("wrote", len(cases), "cases:", ", ".join(c["name"] for c in cases))
