"""The allocator's debug aids behind the C ABI (crates/fe-cuda/src/lib.rs:213-228, 299-343): new memory is zeroed unless
FE_ZERO_ALLOC=0, and with FE_CANARY=1 every allocation has a 64 KB tail of 0xA5 whose damage fe_hip_canary_tails
reports. The switches are read once per process, so each case runs in a process of its own."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import ctypes as C, sys
sys.path.insert(0, %r)
from ferrite_amd import _lib
lib = _lib.lib()
_lib.check(lib.fe_hip_init(0))

class Tail(C.Structure):
    _fields_ = [("base", C.c_uint64), ("bytes", C.c_size_t), ("first", C.c_size_t), ("damaged", C.c_size_t)]

def tails():
    out, n = (Tail * 8)(), C.c_size_t(0)
    _lib.check(lib.fe_hip_canary_tails(C.cast(out, C.c_void_p), 8, C.byref(n)))
    return [(t.base, t.bytes, t.first, t.damaged) for t in out[:min(n.value, 8)]], n.value

p, q = C.c_uint64(0), C.c_uint64(0)
_lib.check(lib.fe_hip_malloc(C.byref(p), 1000))
_lib.check(lib.fe_hip_malloc(C.byref(q), 4096))
host = (C.c_uint8 * 1000)(*([7] * 1000))
_lib.check(lib.fe_hip_memcpy_dtoh(C.cast(host, C.c_void_p), p.value, 1000))
print("zeroed", all(b == 0 for b in host))
print("canary", lib.fe_hip_canary_on())
print("clean", tails())
if lib.fe_hip_canary_on():
    # 8 bytes written 16 bytes past the end of the first buffer: inside its own tail, so nothing faults
    _lib.check(lib.fe_hip_memset_d8(p.value + 1000 + 16, 0x11, 8, None))
    _lib.check(lib.fe_hip_synchronize())
    t, n = tails()
    print("damaged", n, [(b - p.value, size, first, bad) for b, size, first, bad in t])
    _lib.check(lib.fe_hip_free(p.value))
    print("after free", tails())
""" % ROOT


def run_child(env):
    e = dict(os.environ)
    e.pop("FE_CANARY", None)
    e.pop("FE_ZERO_ALLOC", None)
    e.update(env)
    r = subprocess.run([sys.executable, "-c", CHILD], env=e, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stdout


def test_new_memory_is_zeroed_and_the_canary_is_off_by_default():
    out = run_child({})
    assert "zeroed True" in out and "canary 0" in out and "clean ([], 0)" in out


def test_canary_reports_a_write_past_the_end():
    out = run_child({"FE_CANARY": "1"})
    assert "zeroed True" in out and "canary 1" in out and "clean ([], 0)" in out
    assert "damaged 1 [(0, 1000, 16, 8)]" in out
    assert "after free ([], 0)" in out
