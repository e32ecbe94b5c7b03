"""The dump format and its comparison, without a GPU."""
import numpy as np
import pytest

from sonicboom_amd.engine.trace import DumpWriter, compare, read_dump


def test_dump_round_trip_and_comparison(tmp_path):
    a = np.array([[1.0, -2.5, 3.25e-8], [0.0, 1e20, -7.0]], np.float32)
    with DumpWriter(str(tmp_path / "a.dump"), "first") as w:
        w("embedding", a)
        w("entry0.after mixer", a * 2)          # a name may hold spaces
        w("empty", np.zeros((0,), np.float32))
        w("entry0.after mixer", a * 3)          # and may come twice: matched by occurrence
    got = read_dump(str(tmp_path / "a.dump"))
    assert [n for n, _ in got] == ["embedding", "entry0.after mixer", "empty", "entry0.after mixer"]
    assert np.array_equal(got[0][1], a.reshape(-1)) and np.array_equal(got[3][1], (a * 3).reshape(-1))
    text = (tmp_path / "a.dump").read_text().splitlines()
    assert text[0] == "# first" and text[1] == "@ embedding f32 6 1 1 1" and text[2] == "1"
    rows, first_bad, only_ref, only_cand = compare(got, got)
    assert first_bad is None and not only_ref and not only_cand and all(r[5] for r in rows)
    other = [(n, v.copy()) for n, v in got]
    other[1][1][1] *= 1.001                      # a relative error of 1e-3 in the first of the two
    other.append(("extra", np.ones(2, np.float32)))
    rows, first_bad, only_ref, only_cand = compare(got, other[1:], tol=1e-4)
    assert first_bad == "entry0.after mixer" and only_ref == ["embedding"] and only_cand == ["extra"]
    assert [r[5] for r in rows] == [False, True, True]
    assert abs(rows[0][3] - 1e-3) < 1e-5         # |a-b| / max(|a|, |b|)
    # near zero the relative error is large and the absolute one decides
    z = [("t", np.array([1e-9], np.float32))], [("t", np.array([2e-9], np.float32))]
    assert compare(*z)[1] is None
    (tmp_path / "bad.dump").write_text("@ x f32 3 1 1 1\n1\n2\n")
    with pytest.raises(ValueError, match="announces 3"):
        read_dump(str(tmp_path / "bad.dump"))
