"""Writes tests/golden/spec_manifest.json: every `it(` spec of the six op test files of the reference
that exercise this path, with the place in this repository's tests that carries it, or the reason why
nothing does. tests/test_spec_manifest.py fails on a spec without either, and (when the reference is
there to read) on a manifest that no longer matches the test files.

Classes:
  golden       inputs and expected values in tests/golden/<file>.json (written by make_fixtures.py)
  hand-values  the same, transcribed by hand into hand_transcribed.json (make_hand_fixtures.py)
  hand-js      a spec about the form of a call, transcribed into tests/js/hand_specs.js
  error-path   a spec that expects a throw, transcribed into tests/js/error_specs.js
  gradient     tf.grad / tf.grads / tf.valueAndGrad specs: the path is inference, there is no tape
(The tf.dot and tf.outerProduct specs of mat_mul_test.ts are compositions that end in BatchMatMul; their
value specs are in hand_specs.js and their throwing ones in error_specs.js, like the matMul specs'.)

Run:  python tests/golden/make_spec_manifest.py        (needs /root/reference to read the test files)
"""
import json
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
REF = os.environ.get("TFJS_REFERENCE", "/root/reference")
OUT = os.path.join(HERE, "spec_manifest.json")

TEST_FILES = {
    "tfjs-core/src/ops/fused/fused_mat_mul_test.ts": "fused_mat_mul.json",
    "tfjs-core/src/ops/fused/fused_conv2d_test.ts": "fused_conv2d.json",
    "tfjs-core/src/ops/fused/fused_depthwise_conv2d_test.ts": "fused_depthwise_conv2d.json",
    "tfjs-core/src/ops/mat_mul_test.ts": "mat_mul.json",
    "tfjs-core/src/ops/conv2d_test.ts": "conv2d.json",
    "tfjs-core/src/ops/depthwise_conv2d_test.ts": "depthwise_conv2d.json",
}

SPEC = re.compile(r"^\s*(?:it|fit|xit)\(\s*$|^\s*(?:it|fit|xit)\(\s*['`\"]")
SUITE = re.compile(r"^\s*describe\w*\(\s*['`\"]([^'`\"]*)")
GRADIENT_CALL = re.compile(r"\btf\.(grad|grads|valueAndGrad|valueAndGrads)\b")


def read_specs(rel_path):
    """[(line of `it(`, last line, title, suite title, body text)] of one test file."""
    lines = open(os.path.join(REF, rel_path)).read().split("\n")
    specs, suite = [], ""
    for i, text in enumerate(lines):
        m = SUITE.match(text)
        if m:
            suite = m.group(1)
        if not SPEC.match(text):
            continue
        # the spec runs to the line where the parenthesis opened by `it(` closes
        depth, j, quote = 0, i, None
        done = False
        while j < len(lines) and not done:
            k = 0
            row = lines[j]
            while k < len(row):
                ch = row[k]
                if quote:
                    if ch == "\\":
                        k += 1
                    elif ch == quote:
                        quote = None
                elif ch in "'\"`":
                    quote = ch
                elif ch == "/" and row[k:k + 2] == "//":
                    break
                elif ch == "(":
                    depth += 1
                elif ch == ")":
                    depth -= 1
                    if depth == 0:
                        done = True
                        break
                k += 1
            j += 1
        body = "\n".join(lines[i:j])
        title = "".join(re.findall(r"'((?:[^'\\]|\\.)*)'", body.split("=>")[0])) or \
            "".join(re.findall(r"`([^`]*)`", body.split("=>")[0]))
        specs.append((i + 1, j, title, suite, body))
    return specs


def ranges_of(sources, rel_path):
    out = []
    for s in sources:
        path, _, span = s.rpartition(":")
        if path != rel_path:
            continue
        first, _, last = span.partition("-")
        out.append((int(first), int(last or first)))
    return out


def js_spec_lines(js_file, rel_path):
    """Lines named by `at: O + '<file>:<line>'` entries of a tests/js spec table."""
    text = open(os.path.join(HERE, "..", "js", js_file)).read()
    tail = rel_path.split("tfjs-core/src/ops/")[1]
    return {int(n) for n in re.findall(r"at: O \+ '%s:(\d+)'" % re.escape(tail), text)}


def covered(line, last, ranges):
    # a fixture's range starts at the `it(` line, or a blank line or two above it
    return any(first <= line <= first + 2 and abs(end - last) <= 2 for first, end in ranges) or \
        any(first <= line <= end and first >= line - 2 for first, end in ranges)


def build():
    hand = json.load(open(os.path.join(HERE, "hand_transcribed.json")))
    hand_sources = [c["source"] for group in hand.values() for c in group]
    manifest = []
    for rel_path, fixture in TEST_FILES.items():
        golden = json.load(open(os.path.join(HERE, fixture)))
        golden_ranges = ranges_of([c["source"] for c in golden["cases"]], rel_path)
        hand_ranges = ranges_of(hand_sources, rel_path)
        error_lines = js_spec_lines("error_specs.js", rel_path)
        hand_js_lines = js_spec_lines("hand_specs.js", rel_path)
        for line, last, title, suite, body in read_specs(rel_path):
            entry = {"file": rel_path, "line": line, "last_line": last, "suite": suite, "title": title}
            if line in error_lines:
                entry.update({"class": "error-path", "covered_by": "tests/js/error_specs.js"})
            elif line in hand_js_lines:
                entry.update({"class": "hand-js", "covered_by": "tests/js/hand_specs.js"})
            elif covered(line, last, golden_ranges):
                entry.update({"class": "golden", "covered_by": "tests/golden/" + fixture})
            elif covered(line, last, hand_ranges):
                entry.update({"class": "hand-values", "covered_by": "tests/golden/hand_transcribed.json"})
            elif GRADIENT_CALL.search(body) or "gradient" in suite.lower():
                entry.update({"class": "gradient", "covered_by": None})
            else:
                entry.update({"class": "unaccounted", "covered_by": None})
            manifest.append(entry)
    return manifest


def main():
    manifest = build()
    counts = {}
    for e in manifest:
        counts[e["class"]] = counts.get(e["class"], 0) + 1
    with open(OUT, "w") as f:
        json.dump({"counts": counts, "specs": manifest}, f, indent=0)
        f.write("\n")
    print(counts)
    for e in manifest:
        if e["class"] == "unaccounted":
            print("unaccounted: %s:%d %s" % (e["file"], e["line"], e["title"]))


if __name__ == "__main__":
    main()
