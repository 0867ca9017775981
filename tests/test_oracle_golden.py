"""The committed vectors of tests/golden/path_vectors.npz against the oracle as it is now (CPU). The file was written by
tests/golden/make_golden.py from the oracle; a change of the oracle that alters one bit of them fails here."""
import importlib.util
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def test_oracle_reproduces_the_committed_vectors(oracle):
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    now = mod.vectors()
    gold = np.load(os.path.join(HERE, "golden", "path_vectors.npz"))
    assert sorted(gold.files) == sorted(now)
    for name in gold.files:
        a, b = gold[name], np.asarray(now[name])
        assert a.shape == b.shape and a.dtype == b.dtype, name
        assert a.tobytes() == np.ascontiguousarray(b).tobytes(), name


def test_known_answers_are_in_the_file():
    """decode_mul1 of states 0, 1 and 0xffff (closed form: 0xc2e8, 0x3921, 0xb936)."""
    gold = np.load(os.path.join(HERE, "golden", "path_vectors.npz"))
    by = dict(zip(gold["mul1_states"].tolist(), gold["mul1_f16"].tolist()))
    assert by[0] == 0xC2E8 and by[1] == 0x3921 and by[0xFFFF] == 0xB936
