"""Saved variable environments (CPU side): the text written and read by libag_host.so is the
reference's format -- serde_json of {"array_list":[{"v":1,"dim":[..],"data":[..]},..],
"name_to_id":{"ns\\u0001name":id,..}} (src/variable.rs:470-480, 549-598; ndarray's serde form,
version 1).  Nothing here touches a device: files are parsed and written in host memory.

What pins the format: the reference's own tests only round-trip (src/variable.rs:811-866, mirrored on
the GPU in test_gpu_graph.py); the byte layout follows the published formats of serde_json and ndarray's
`serde` feature, written out by hand in tests/golden/variable_env_f32.json.  A file written by the
reference itself cannot be produced here (no Rust toolchain), so byte equality with one is unchecked.
Number printing is checked against numpy's shortest-round-trip digits, not against this code's own
formatter.
"""
import json
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "variable_env_f32.json")


@pytest.fixture(scope="module")
def G():
    from __graft_entry__ import load_package

    load_package()
    import rust_autograd_amd.graph as graph

    graph.lib()
    return graph


def rewrite(G, tmp_path, text, name="in.json"):
    src, dst = tmp_path / name, tmp_path / ("out_" + name)
    src.write_text(text)
    G.rewrite_saved_environment(str(src), str(dst))
    return dst.read_text()


def test_golden_file_is_reproduced_byte_for_byte(G, tmp_path):
    text = open(GOLDEN).read()
    assert rewrite(G, tmp_path, text) == text


def test_golden_file_values(G):
    # the fixture read with Python's own JSON reader says what the numbers are meant to be
    doc = json.load(open(GOLDEN))
    assert [a["dim"] for a in doc["array_list"]] == [[2, 3], [], [5], [0, 2]]
    assert doc["name_to_id"] == {"\x01a": 0, "\x01b": 1, "adam\x01am": 2}
    got = np.array(doc["array_list"][2]["data"], dtype=np.float64).astype(np.float32)
    want = np.array([1e13, 1e12, np.finfo(np.float32).max, np.float32(1e-45), -0.0], dtype=np.float32)
    assert got.tobytes() == want.tobytes()


def test_any_layout_serde_json_accepts_is_read(G, tmp_path):
    # whitespace, field order inside an array, integers and exponents for floats, escapes in names,
    # a field the struct does not have
    text = """
    { "extra": [1, {"k": null}, "s\\n"],
      "name_to_id": { "\\u0001w\\"1": 1, "ns\\u0001caf\\u00e9": 0 },
      "array_list": [ { "data": [1, 2E0, -3.5e+0, 4.25], "dim": [2, 2], "v": 1 },
                      { "dim": [1], "v": 1, "data": [0.30000001192092896] } ] }
    """
    out = rewrite(G, tmp_path, text)
    assert out == ('{"array_list":[{"v":1,"dim":[2,2],"data":[1.0,2.0,-3.5,4.25]},{"v":1,"dim":[1],"data":[0.3]}],'
                   '"name_to_id":{"\\u0001w\\"1":1,"ns\\u0001café":0}}')


def shortest_digits(v):
    s = np.format_float_scientific(np.float32(v), unique=True, trim="-")
    return s.split("e")[0].replace(".", "").replace("-", "").rstrip("0") or "0"


def test_numbers_are_shortest_round_trip_and_always_floats(G, tmp_path):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    vals = bits.view(np.float32)
    vals = vals[np.isfinite(vals)]
    extra = np.array([0.0, 1.0, 0.1, 1e-7, 1e-6, 9.999999e12, 1e13, 1.5e13, 123456.79, 16777216.0, 5e-324, 1e-38],
                     dtype=np.float32)
    vals = np.concatenate([vals, extra, rng.standard_normal(5000).astype(np.float32)])
    doc = {"array_list": [{"v": 1, "dim": [len(vals)], "data": [float(v) for v in vals]}], "name_to_id": {}}
    out = rewrite(G, tmp_path, json.dumps(doc))
    tokens = out[out.index('"data":[') + 8:out.index("]}]")].split(",")
    assert len(tokens) == len(vals)
    back = np.array([float(t) for t in tokens], dtype=np.float64).astype(np.float32)
    assert back.tobytes() == vals.tobytes()                      # bit-exact, signed zeros included
    for tok, v in zip(tokens, vals):
        assert re.fullmatch(r"-?\d+\.\d+(e-?\d+)?|-?\d+e-?\d+", tok), tok   # never a bare integer
        digits = re.sub(r"e.*", "", tok).replace(".", "").replace("-", "").strip("0") or "0"
        assert len(digits) <= len(shortest_digits(v)), (tok, v)   # no longer than the shortest repr


@pytest.mark.parametrize("value,text", [
    (1.0, "1.0"), (-2.5, "-2.5"), (0.1, "0.1"), (12.34, "12.34"), (0.001234, "0.001234"), (0.00001, "0.00001"),
    (1e-6, "0.000001"), (1e-7, "1e-7"), (1.234e-7, "1.234e-7"), (1e12, "1000000000000.0"), (1e13, "1e13"),
    (1.234e33, "1.234e33"), (1e30, "1e30"), (16777216.0, "16777216.0"), (3.4028235e38, "3.4028235e38"),
])
def test_number_layout_known_answers(G, tmp_path, value, text):
    # plain notation while the point stays within 13 digits right / 5 zeros left of the digits
    doc = {"array_list": [{"v": 1, "dim": [1], "data": [value]}], "name_to_id": {}}
    out = rewrite(G, tmp_path, json.dumps(doc))
    assert out == '{"array_list":[{"v":1,"dim":[1],"data":[%s]}],"name_to_id":{}}' % text


def test_a_value_too_large_for_f32_becomes_infinite_and_is_written_as_null(G, tmp_path):
    out = rewrite(G, tmp_path, '{"array_list":[{"v":1,"dim":[2],"data":[1e300,-1e300]}],"name_to_id":{}}')
    assert '"data":[null,null]' in out


@pytest.mark.parametrize("text,message", [
    ('{"array_list":[],"name_to_id":{}', "EOF"),
    ('{"array_list":[]}', "missing field `name_to_id`"),
    ('{"name_to_id":{}}', "missing field `array_list`"),
    ('{"array_list":[{"v":2,"dim":[1],"data":[1.0]}],"name_to_id":{}}', "unknown array version"),
    ('{"array_list":[{"v":1,"dim":[2],"data":[1.0]}],"name_to_id":{}}', "data and dimension must match in size"),
    ('{"array_list":[{"v":1,"dim":[1]}],"name_to_id":{}}', "missing field `data`"),
    ('{"array_list":[{"v":1,"dim":[1],"data":[1.0],"x":0}],"name_to_id":{}}', "unknown field `x`"),
    ('{"array_list":[{"v":1,"dim":[1],"data":[null]}],"name_to_id":{}}', "null"),
    ('{"array_list":[{"v":1,"dim":[-1],"data":[]}],"name_to_id":{}}', "negative"),
    ('{"array_list":[{"v":1,"dim":[1.5],"data":[1.0]}],"name_to_id":{}}', "floating point"),
    ('{"array_list":[],"name_to_id":{"a":"b"}}', "expected value"),
    ('{"array_list":[],"name_to_id":{}} x', "trailing characters"),
    ('{"array_list":[{"v":1,"dim":[1],"data":[01]}],"name_to_id":{}}', "expected"),
])
def test_malformed_files_are_errors_not_crashes(G, tmp_path, text, message):
    with pytest.raises(G.PersistError, match=re.escape(message)):
        rewrite(G, tmp_path, text)


def test_missing_file_is_an_error(G, tmp_path):
    with pytest.raises(G.PersistError, match="cannot open"):
        G.rewrite_saved_environment(str(tmp_path / "nope.json"), str(tmp_path / "out.json"))
    with pytest.raises(G.PersistError, match="cannot open"):
        G.VariableEnvironment.load(str(tmp_path / "nope.json"))
