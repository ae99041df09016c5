"""Writes tests/golden/highrank_kats.json: inputs and expected gradients that the
reference's own tests hold as literals (test/tool/CrossTesting.hs: t16, t16b,
t128; test/simplified/TestHighRankSimplified.hs: testFoo, testFooD,
testFooBuild0, testFooBuildOut; test/simplified/TestConvSimplified.hs: the
testKonst5* / testKonstNot* gradients of conv2dPreserving on fixed data).  Reads the reference's files as text; nothing is executed.
Run from the repository root with the reference at /root/reference."""
import json
import os
import re

REF = "/root/reference/test"
NUM = r"-?\d+(?:\.\d+)?(?:e-?\d+)?"


def numbers(text):
    return [float(x) for x in re.findall(NUM, text)]


def literal_lists(block):
    """every `[shape] [values]` pair of ringestData literals in block"""
    out = []
    for m in re.finditer(r"ringestData\s*\(?(?:fromList\s*)?\[([\d,\s]+)\]\)?\s*\[([^\]]+)\]", block):
        out.append(([int(x) for x in re.findall(r"\d+", m.group(1))], numbers(m.group(2))))
    return out


def block(text, start, end):
    i = text.index(start)
    return text[i:text.index(end, i + len(start))]


cross = open(os.path.join(REF, "tool/CrossTesting.hs")).read()
high = open(os.path.join(REF, "simplified/TestHighRankSimplified.hs")).read()

t16 = literal_lists(block(cross, "\nt16 =", "\nt16b ::"))[0]
t128 = literal_lists(block(cross, "\nt128 =", "\nt128b ::"))[0]
t16b = literal_lists(block(cross, "\nt16b =", "\nt48 ::"))[0]
conv = open(os.path.join(REF, "simplified/TestConvSimplified.hs")).read()
conv = conv[conv.index("\n-- with data t16\n"):conv.index("\n-- with data t128b and t128c\n")]
conv_kats = {}
for m in re.finditer(r"\n(testKonst\w+) =\n(.*?)(?=\n\n|\Z)", conv, re.S):
    name, body = m.group(1), m.group(2)
    exp = literal_lists(body)[0]
    fn = re.search(r"rev' @Double @4 (conv2d\w+)", body).group(1)
    rep = re.search(r"rreplicate0N \[([\d, ]+)\] 5\)\)", body)
    if rep:
        shape = [int(x) for x in re.findall(r"\d+", rep.group(1))]
        arg = {"shape": shape, "fill": 5.0}
    else:
        ing = re.search(r"ringestData \[([\d, ]+)\] \[37, 36 \.\. -10\]", body)
        shape = [int(x) for x in re.findall(r"\d+", ing.group(1))]
        arg = {"shape": shape, "enum_from_then_to": [37, 36, -10]}
    conv_kats[name] = {"epsilon": float(re.search(r"assertEqualUpToEpsilon' (\S+)", body).group(1)), "function": fn, "argument": arg,
                       "expected_shape": exp[0], "expected": exp[1]}
assert len(conv_kats) == 18, sorted(conv_kats)
foo = literal_lists(block(high, "\ntestFoo =", "\nbar ::"))
food = literal_lists(block(high, "\ntestFooD =", "\nfooBuild0 ::"))
build0 = literal_lists(block(high, "\ntestFooBuild0 =", "\nfooBuildOut"))
buildout = literal_lists(block(high, "\ntestFooBuildOut =", "\nfooBuild2"))
assert len(foo) == 3 and len(food) == 3 and all(len(v) == 16 for _, v in foo) and all(len(v) == 128 for _, v in food)

out = {
    "_source": "literals of test/tool/CrossTesting.hs (t16 :457-458, t128 :466-467) and test/simplified/TestHighRankSimplified.hs "
               "(testFoo, testFooD, testFooBuild0, testFooBuildOut); written by make_highrank_kats.py",
    "t16": {"shape": t16[0], "values": t16[1]},
    "t128": {"shape": t128[0], "values": t128[1]},
    "t16b": {"shape": t16b[0], "values": t16b[1]},
    "conv": conv_kats,
    "testFoo": {"dtype": "f32", "epsilon": 1e-3, "inputs": ["t16", "t16", "t16"], "expected": [v for _, v in foo]},
    "testFooD": {"dtype": "f64", "epsilon": 1e-10, "inputs": ["t128", 0.7, "t128"], "expected": [v for _, v in food]},
    "testFooBuild0": {"input": "t16", "expected": build0[0][1]},
    "testFooBuildOut": {"input": "t16", "expected": buildout[0][1]},
}
json.dump(out, open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "highrank_kats.json"), "w"), indent=1)
print({k: (len(v["expected"]) if isinstance(v, dict) and "expected" in v else None) for k, v in out.items()}, sorted(conv_kats))
