"""Every spec of the reference's six op test files for this path is accounted for: carried by a
fixture or a transcribed JavaScript spec that the suites here run, or classed out of scope with a
reason (gradients only: no tape on an inference path). The manifest is data written by tests/golden/make_spec_manifest.py."""
import importlib.util
import json
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
REFERENCE = os.environ.get("TFJS_REFERENCE", "/root/reference")
CARRIED = {"golden", "hand-values", "hand-js", "error-path"}
OUT_OF_SCOPE = {"gradient"}
EXPECTED_TOTALS = {  # `it(` specs per file of the reference at the surveyed commit
    "tfjs-core/src/ops/fused/fused_mat_mul_test.ts": 21,
    "tfjs-core/src/ops/fused/fused_conv2d_test.ts": 54,
    "tfjs-core/src/ops/fused/fused_depthwise_conv2d_test.ts": 13,
    "tfjs-core/src/ops/mat_mul_test.ts": 72,
    "tfjs-core/src/ops/conv2d_test.ts": 44,
    "tfjs-core/src/ops/depthwise_conv2d_test.ts": 41,
}


def manifest():
    with open(os.path.join(GOLDEN, "spec_manifest.json")) as f:
        return json.load(f)


def generator():
    spec = importlib.util.spec_from_file_location("make_spec_manifest", os.path.join(GOLDEN, "make_spec_manifest.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def test_no_spec_is_unaccounted_and_every_file_is_complete():
    specs = manifest()["specs"]
    stray = [e for e in specs if e["class"] not in CARRIED | OUT_OF_SCOPE]
    assert not stray, "specs neither carried nor classed: %s" % [(e["file"], e["line"]) for e in stray]
    per_file = {}
    for e in specs:
        per_file[e["file"]] = per_file.get(e["file"], 0) + 1
    assert per_file == EXPECTED_TOTALS
    carried = sum(1 for e in specs if e["class"] in CARRIED)
    # every forward, shape and error spec of the six files, tf.dot / tf.outerProduct included: all but the gradient ones
    assert carried == len(specs) - sum(1 for e in specs if e["class"] in OUT_OF_SCOPE) == 207
    assert not [e for e in specs if e["class"] == "other-op"]


def test_every_carried_spec_points_at_something_the_suites_run():
    gen = generator()
    hand = json.load(open(os.path.join(GOLDEN, "hand_transcribed.json")))
    hand_sources = [c["source"] for group in hand.values() for c in group]
    for e in manifest()["specs"]:
        if e["class"] == "golden":
            cases = json.load(open(os.path.join(HERE, "..", e["covered_by"])))["cases"]
            ranges = gen.ranges_of([c["source"] for c in cases], e["file"])
            assert gen.covered(e["line"], e["last_line"], ranges), e
        elif e["class"] == "hand-values":
            assert gen.covered(e["line"], e["last_line"], gen.ranges_of(hand_sources, e["file"])), e
        elif e["class"] in ("hand-js", "error-path"):
            assert e["line"] in gen.js_spec_lines(os.path.basename(e["covered_by"]), e["file"]), e


def test_transcribed_js_specs_name_real_specs_only():
    """An `at:` key of the JavaScript spec tables that matches no `it(` line would be a spec nobody wrote."""
    gen = generator()
    by_file = {}
    for e in manifest()["specs"]:
        by_file.setdefault(e["file"], set()).add(e["line"])
    for js in ("error_specs.js", "hand_specs.js"):
        for rel_path, lines in by_file.items():
            assert gen.js_spec_lines(js, rel_path) <= lines, (js, rel_path)
    # and the two tables are wired into both JavaScript tiers
    for tier in ("cpu_tests.js", "gpu_tests.js"):
        text = open(os.path.join(HERE, "js", tier)).read()
        assert re.search(r"require\('./error_specs'\)", text) and re.search(r"require\('./hand_specs'\)", text), tier


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "tfjs-core")), reason="the reference tree is not on this machine")
def test_manifest_matches_the_reference_test_files():
    fresh = generator().build()
    assert fresh == manifest()["specs"], "run tests/golden/make_spec_manifest.py"
