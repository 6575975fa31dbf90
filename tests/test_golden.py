"""The committed fixture of benchmark config 0 (tests/golden/config0_int8.json, made by
tests/golden/make_config0_fixture.py from the CPU oracle): the oracle must still reproduce it bit for
bit, and the HIP path must produce the same bytes without the oracle being run."""
import importlib.util
import json
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = json.load(open(os.path.join(HERE, "golden", "config0_int8.json")))
spec = importlib.util.spec_from_file_location("make_config0_fixture", os.path.join(HERE, "golden", "make_config0_fixture.py"))
gen = importlib.util.module_from_spec(spec)
spec.loader.exec_module(gen)


def test_oracle_reproduces_the_committed_fixture():
    t = gen.compute()
    assert set(t) == set(FIX["sha256"])
    for name, v in t.items():
        assert gen.digest(v) == FIX["sha256"][name], name
        assert gen.corner(v) == FIX["corner"][name], name


@pytest.mark.gpu
def test_hip_path_reproduces_the_committed_fixture():
    import dax_amd.ops as ops
    from oracle import daxq_oracle as O   # inputs only: the seeded generator of the workload

    c = FIX["config"]
    x, w, b = O.make_inputs(c["m"], c["k"], c["n"], seed=c["seed"])
    assert gen.digest(x) == FIX["sha256"]["x"] and gen.digest(w) == FIX["sha256"]["w"]
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    lo, hi = ops.row_minmax(wd)
    sw = ops.scale_from_minmax(lo, hi, 127.0)
    qw = ops.quantize_rows_i8(wd, sw, True)
    xq, sx = ops.act_quant_i8(xd)
    out, acc = ops.linear_i8_acc(xq, sx, qw, sw, bd)
    got = {"qweight": qw[:, :c["k"]], "weight_scale": sw, "xq": xq[:, :c["k"]], "sx": sx, "acc": acc, "out": out}
    sw8 = ops.scale_from_minmax(lo, hi, 448.0)
    xq8, sx8 = ops.act_quant_e4m3(xd)
    got.update({"xq_e4m3": xq8[:, :c["k"]], "sx_e4m3": sx8, "qweight_e4m3": ops.quantize_rows_e4m3(wd, sw8), "weight_scale_e4m3": sw8})
    for name, v in got.items():
        assert gen.digest(v.contiguous()) == FIX["sha256"][name], name
