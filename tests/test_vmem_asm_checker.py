"""The build-time assembly checker (bmtrain_amd/csrc/check_vmem_asm.py) on known inputs.

Three product kernels place their own `s_waitcnt vmcnt(N)` and issue their vector-memory instructions
from asm statements; what the compiler normally guarantees for them is proved on its assembly output by
that checker at every build.  These tests pin the checker itself: hand-written assembly in the shape of
those loops (tests/fixtures/vmem_*.s; never compiled or run) that is correct must pass, and each of the
three mistakes the checker exists for must be reported:

  * a first-stage wait of vmcnt(5) where vmcnt(4) is needed (the last load of the current register set
    may still be in flight when it is used),
  * a 16-byte store without its `s_nop 1` (the next vector instruction overwrites data the store still reads),
  * a wave that ends with a load in flight.

The shipped kernels' own assembly is checked too when a build has left it next to the sources, and the
generated code of every kernel file must hold no packed-fp32 arithmetic.
"""
import glob
import importlib.util
import os
import re

import pytest

from conftest import ROOT

CSRC = os.path.join(ROOT, "bmtrain_amd", "csrc")
FIXTURES = os.path.join(ROOT, "tests", "fixtures")


def load_checker():
    spec = importlib.util.spec_from_file_location("check_vmem_asm", os.path.join(CSRC, "check_vmem_asm.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def run_checker(path, wanted):
    """[(kernel name, problems)] for every kernel of `path` whose label contains one of `wanted`."""
    chk = load_checker()
    lines = open(path).read().split("\n")
    out = []
    for i, line in enumerate(lines):
        m = re.match(r"^(\w+):\s*;\s*@", line)
        if m and any(w in m.group(1) for w in wanted):
            problems, n_inst, loads, waits = chk.check(lines, i, m.group(1))
            out.append((m.group(1), problems, n_inst, loads, waits))
    return out


def test_a_correct_pipeline_is_accepted():
    (name, problems, n_inst, loads, waits), = run_checker(os.path.join(FIXTURES, "vmem_good_pipeline.s"), ["good_pipeline"])
    assert problems == []
    assert loads == 12 and waits == 3 and n_inst > 50      # the whole loop was parsed, not an empty kernel


def test_a_too_weak_first_wait_is_reported():
    (name, problems, *_), = run_checker(os.path.join(FIXTURES, "vmem_weak_first_wait.s"), ["weak_first_wait"])
    assert problems, "vmcnt(5) after four loads leaves the previous set's last load in flight"
    text = "\n".join(problems)
    assert "while a load into it is in flight" in text
    # exactly the registers of the last load of set A (v[12:15]) are the ones in flight, nothing else
    touched = set()
    for p in problems:
        m = re.search(r"v\[([0-9, ]+)\] while a load", p)
        assert m, p
        touched.update(int(x) for x in m.group(1).split(","))
    assert touched == {12, 13, 14, 15}


def test_a_wide_store_without_its_nop_is_reported():
    (name, problems, *_), = run_checker(os.path.join(FIXTURES, "vmem_store_without_nop.s"), ["store_without_nop"])
    assert len(problems) == 8                                # every one of the eight 16-byte stores
    assert all("overwrites data of `global_store_dwordx4" in p and "0 wait state(s)" in p for p in problems)


def test_a_wave_that_ends_with_a_load_in_flight_is_reported():
    (name, problems, *_), = run_checker(os.path.join(FIXTURES, "vmem_ends_with_load_in_flight.s"),
                                        ["ends_with_load_in_flight"])
    assert len(problems) == 1 and "the wave ends with loads in flight" in problems[0]


def test_the_bad_fixtures_differ_from_the_good_one_only_in_the_mistake():
    """Guards the fixtures themselves: each bad file is the good one with one kind of line changed."""
    def body(name):
        return [l for l in open(os.path.join(FIXTURES, name)).read().split("\n") if l.startswith("\t")]   # instructions
    good = body("vmem_good_pipeline.s")
    weak = body("vmem_weak_first_wait.s")
    assert len(weak) == len(good)
    assert [(a, b) for a, b in zip(good, weak) if a != b] == [("\ts_waitcnt vmcnt(4)", "\ts_waitcnt vmcnt(5)")]
    assert body("vmem_store_without_nop.s") == [l for l in good if l != "\ts_nop 1"]
    assert body("vmem_ends_with_load_in_flight.s") == [l for l in good if l != "\ts_waitcnt vmcnt(0)"]


SHIPPED = (("adam.device.s", ["adam_stream_kernel", "adam_stream_multi_kernel"], 12),   # (2 flavours x 2 counter homes + 2 multi) x counters fixed / in turn
           ("cross_entropy.device.s", ["ce_flat_stream_kernel"], 16))   # 2 types x 2 operations x rows on / off the vector grid x counters fixed / in turn


@pytest.mark.parametrize("filename,wanted,expect", SHIPPED)
def test_the_shipped_kernels_pass(filename, wanted, expect):
    path = os.path.join(CSRC, filename)
    if not os.path.exists(path):
        pytest.skip("no build has left %s next to the sources" % filename)
    results = run_checker(path, wanted)
    assert len(results) == expect                            # every instantiation of each kernel
    for name, problems, n_inst, loads, waits in results:
        assert problems == [], name
        assert loads >= 12 and waits >= 3


def test_no_packed_fp32_arithmetic_in_the_generated_code():
    files = sorted(glob.glob(os.path.join(CSRC, "*.device.s")))
    if not files:
        pytest.skip("no build has left device assembly next to the sources")
    assert {os.path.basename(f) for f in files} >= {"adam.device.s", "has_inf_nan.device.s", "cross_entropy.device.s"}
    for f in files:
        hits = [l for l in open(f) if re.search(r"\bv_pk_[a-z0-9]+_f32\b", l)]
        assert hits == [], (f, hits[:3])
