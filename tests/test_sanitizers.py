"""Host-side sanitizer runs (CPU only): the AddressSanitizer + UndefinedBehaviorSanitizer builds of `make -C tests/cpp asan`.

* tests/bin/oracle_sanitize walks every function of the CPU oracle over awkward shapes;
* tests/bin/test_core_api_asan host runs the argument checks and shape rules behind the dlprim::core headers;
* tests/bin/net_forward_asan parses JSON documents (well formed and malformed), and plans every test network and the three
  benchmark networks on a CPU context: the JSON reader, shape inference, the graph rewrites and the memory planner of
  include/dlprim/net.hpp with every heap access and signed overflow checked.
A sanitizer report makes the binary exit non-zero (-fno-sanitize-recover, ASan's default abort)."""
import json
import os
import subprocess

import pytest

import test_net
from dlprimitives_amd import netfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "bin")
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")


def run(name, *args, ok=True):
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        pytest.fail("tests/bin/%s is not built: run `make -C tests/cpp asan` (or __graft_entry__.build())" % name)
    r = subprocess.run([path] + [str(a) for a in args], capture_output=True, text=True, timeout=600, env=ENV)
    assert "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]
    if ok:
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return r


def test_oracle_under_sanitizers():
    assert "ok" in run("oracle_sanitize").stdout


def test_core_api_host_checks_under_sanitizers():
    run("test_core_api_asan", "host")


@pytest.mark.parametrize("doc", test_net.JSON_DOCS, ids=range(len(test_net.JSON_DOCS)))
def test_json_reader_under_sanitizers(tmp_path, doc):
    p = tmp_path / "d.json"
    p.write_text(json.dumps(doc, ensure_ascii=False), encoding="utf-8")
    assert json.loads(run("net_forward_asan", "json", p).stdout) == doc


@pytest.mark.parametrize("text", ["{", "[1,]", '{"a" 1}', '{"a": tru}', '"open', "[1] x", "", '{"a": 1e}', '"\\u12"', "nul", '"\\ud800"', '"\\ud800\\u0041"', '"\\udc00 x"', "[" * 2000, "-", "1e999"])
def test_json_reader_rejects_malformed_under_sanitizers(tmp_path, text):
    p = tmp_path / "bad.json"
    p.write_text(text)
    r = run("net_forward_asan", "json", p, ok=False)
    assert r.returncode in (0, 1)  # an error message or a value, never a sanitizer report or a crash
    if "\\ud" in text:
        assert r.returncode == 1 and "surrogate" in r.stderr  # unpaired surrogates are refused, as the reference's decoder refuses them


NETS = dict(test_net.NETS)
NETS.update({"resnet18_b16_224": (lambda: netfile.resnet18(16, 224, 1000), 0), "resnet50_b16_224": (lambda: netfile.resnet50(16, 224, 1000), 0),
             "mobilenet_v2_b16_224": (lambda: netfile.mobilenet_v2(16, 224, 1000), 0)})


@pytest.mark.parametrize("flags", [(), ("nofuse",), ("keep",)], ids=["default", "nofuse", "keep"])
@pytest.mark.parametrize("net", list(NETS))
def test_net_plan_under_sanitizers(tmp_path, net, flags):
    b = NETS[net][0]()
    p = tmp_path / "net.json"
    p.write_text(json.dumps(b.doc, indent=1))
    out = run("net_forward_asan", "plan", p, *flags).stdout
    assert out.startswith("operators ")


def test_net_plan_errors_under_sanitizers(tmp_path):
    """networks the planner must refuse: the refusal is an exception, not an out-of-bounds access on the way to it"""
    b = netfile.NetBuilder("data", (2, 3, 8, 8))
    b.conv("data", "c", 4, 3, 1, 1, bias=True)
    b.output("c")
    good = b.doc
    broken = []
    d = json.loads(json.dumps(good)); d["operators"][0]["inputs"] = ["nowhere"]; broken.append(d)
    d = json.loads(json.dumps(good)); d["outputs"] = ["missing"]; broken.append(d)
    d = json.loads(json.dumps(good)); d["operators"][0]["options"]["channels_in"] = 5; broken.append(d)
    d = json.loads(json.dumps(good)); d["operators"][0]["options"]["kernel"] = [9, 9]; d["operators"][0]["options"]["pad"] = [0, 0]; broken.append(d)
    d = json.loads(json.dumps(good)); d["operators"][0]["type"] = "NoSuchOperator"; broken.append(d)
    d = json.loads(json.dumps(good)); d["inputs"][0]["shape"] = [2, 3, 8]; broken.append(d)
    d = json.loads(json.dumps(good)); del d["operators"][0]["options"]["channels_out"]; broken.append(d)
    for i, doc in enumerate(broken):
        p = tmp_path / ("bad%d.json" % i)
        p.write_text(json.dumps(doc))
        r = run("net_forward_asan", "plan", p, ok=False)
        assert r.returncode == 1, (i, r.stdout, r.stderr)
