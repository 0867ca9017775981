"""Python mirror of the reference's fe-exl3 layer API over the C ABI (include/fe_exl3.h).

Names, argument meaning and error behaviour follow crates/fe-exl3/src/{format,linear}.rs and gpu/mod.rs:
`Exl3Tensor` (host container and its layout helpers), `Exl3View`, `DeviceExl3`, `Kernels`, `Plan`, `Dtype`,
`Workspace`, `Linear`. torch tensors hold device memory; every compute call goes to libferrite_amd.so.
"""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass

import numpy as np

from . import _lib
from ._lib import FeError, PlanC, View, check

MUL1 = 0x83DCD12D  # crates/fe-exl3/src/format.rs:14


class Dtype(enum.IntEnum):
    """Activation element type; the Add forms are outputs only (crates/fe-exl3/src/linear.rs:12-31)."""
    Bf16 = 0
    F32 = 1
    Bf16Add = 2
    F32Add = 3


class Exl3Tensor:
    """An EXL3 tensor in host memory (crates/fe-exl3/src/format.rs:16-30): W is [k][n]; trellis = little-endian u32
    words, tile (kt, nt) at [(kt * n/16 + nt) * 8 * bits ..][.. 8 * bits]; suh fp16 bits [k]; svh fp16 bits [n]."""

    def __init__(self, name, k, n, bits, trellis, suh, svh):
        self.name, self.k, self.n, self.bits = name, int(k), int(n), int(bits)
        self.trellis = np.ascontiguousarray(trellis, dtype=np.uint32).reshape(-1)
        self.suh = np.ascontiguousarray(suh, dtype=np.uint16).reshape(-1)
        self.svh = np.ascontiguousarray(svh, dtype=np.uint16).reshape(-1)
        if not 1 <= self.bits <= 8:
            raise ValueError(f"{name}: {bits} bits")  # format.rs:42-44
        if self.k % 16 or self.n % 16 or self.trellis.size != self.k // 16 * (self.n // 16) * self.tile_words():
            raise ValueError(f"{name}: trellis of {self.trellis.size} words for {k}x{n} at {bits} bits")
        if self.suh.size != self.k or self.svh.size != self.n:
            raise ValueError(f"{name}: suh {self.suh.size} svh {self.svh.size} for {k}x{n}")  # format.rs:53-55

    def tile_words(self):
        return 8 * self.bits  # format.rs:60-62

    def tile(self, kt, nt):
        tw = self.tile_words()
        i = (kt * (self.n // 16) + nt) * tw
        return self.trellis[i:i + tw]  # format.rs:64-68

    def strips(self):
        """[n/128][k/16][8][tw]: each 128-column block's K range contiguous (format.rs:70-84)."""
        tw, kt, nt = self.tile_words(), self.k // 16, self.n // 16
        return np.ascontiguousarray(self.trellis.reshape(kt, nt // 8, 8 * tw).transpose(1, 0, 2)).reshape(-1)

    def slice_cols(self, ranges):
        """Column slice (format.rs:86-110): each range 128-aligned; an exact EXL3 tensor of its own."""
        nt, tw = self.n // 16, self.tile_words()
        for a, b in ranges:
            if a % 128 or b % 128 or a >= b or b > self.n:
                raise ValueError(f"{self.name}: column range {a}..{b} not 128-aligned in 0..{self.n}")
        t3 = self.trellis.reshape(self.k // 16, nt, tw)
        trellis = np.concatenate([t3[:, a // 16:b // 16] for a, b in ranges], axis=1)
        svh = np.concatenate([self.svh[a:b] for a, b in ranges])
        return Exl3Tensor(f"{self.name}[cols]", self.k, svh.size, self.bits, trellis, self.suh.copy(), svh)

    def slice_rows(self, k0, k1):
        """Row (input) slice [k0, k1) (format.rs:112-130): the partials of all slices sum to the full output."""
        if k0 % 128 or k1 % 128 or k0 >= k1 or k1 > self.k:
            raise ValueError(f"{self.name}: row range {k0}..{k1} not 128-aligned in 0..{self.k}")
        row_words = self.n // 16 * self.tile_words()
        return Exl3Tensor(f"{self.name}[rows {k0}..{k1}]", k1 - k0, self.n, self.bits,
                          self.trellis[k0 // 16 * row_words:k1 // 16 * row_words].copy(), self.suh[k0:k1].copy(), self.svh.copy())

    def trellis_bytes(self):
        return self.trellis.size * 4  # format.rs:132-135


def value_row(lane, j):
    return 2 * (lane & 3) + (j & 1) + 8 * ((j >> 1) & 1)  # format.rs:148-150


def value_col(lane, j):
    return (lane >> 2) + 8 * (j >> 2)  # format.rs:154-156


@dataclass
class Exl3View:
    """Device pointers of one EXL3 tensor (crates/fe-exl3/src/gpu/mod.rs:15-34)."""
    k: int
    n: int
    bits: int
    trellis: int
    suh: int
    svh: int
    strips: bool

    def strides(self):
        tw = 8 * self.bits
        return (8 * tw, self.k // 16 * 8 * tw) if self.strips else (self.n // 16 * tw, 8 * tw)

    def c(self):
        return View(self.k, self.n, self.bits, self.trellis, self.suh, self.svh, 1 if self.strips else 0)


def _dev(arr, torch_dtype=None):
    import torch
    if arr.dtype == np.uint32:
        return torch.from_numpy(arr.view(np.int32)).cuda()
    if arr.dtype == np.uint16:
        return torch.from_numpy(arr.view(np.int16)).cuda()
    return torch.from_numpy(arr).cuda()


class DeviceExl3:
    """An EXL3 tensor uploaded to device memory (crates/fe-exl3/src/gpu/mod.rs:36-75)."""

    def __init__(self, t: Exl3Tensor, strips: bool):
        _lib.init()
        self.name = t.name
        self.trellis = _dev(t.strips() if strips else t.trellis)
        self.suh = _dev(t.suh)
        self.svh = _dev(t.svh)
        self.view = Exl3View(t.k, t.n, t.bits, self.trellis.data_ptr(), self.suh.data_ptr(), self.svh.data_ptr(), strips)

    @classmethod
    def upload(cls, t):  # stored layout (what reconstruct reads)
        return cls(t, False)

    @classmethod
    def upload_strips(cls, t):  # decode GEMV
        return cls(t, True)


@dataclass
class Plan:
    """Launch plan (crates/fe-exl3/src/linear.rs:33-55)."""
    sk: int
    wk: int = 4
    ver: int = 1
    occ: int = 0

    @staticmethod
    def parse(s: str):
        p = PlanC()
        try:
            check(_lib.lib().fe_exl3_plan_parse(s.encode(), C.byref(p)))
        except FeError:
            return None
        return Plan(p.sk, p.wk, p.ver, p.occ)

    def c(self):
        return PlanC(self.sk, self.wk, self.ver, self.occ)


def default_blocks(cu_count: int) -> int:
    """Programs a GEMV launch aims for: 4 a CU (linear.rs:131-134)."""
    return 4 * cu_count


def _stream(s):
    """A stream argument: None = torch's current stream, a torch stream, a raw handle (int) or a ctypes pointer."""
    if s is None:
        import torch
        s = torch.cuda.current_stream()
    if isinstance(s, C.c_void_p):
        return s
    return C.c_void_p(getattr(s, "cuda_stream", s))


class Kernels:
    """The gfx950 code object of the EXL3 kernels, loaded into the current context (gpu/mod.rs:77-102)."""

    def __init__(self):
        _lib.init()
        self.h = C.c_void_p()
        check(_lib.lib().fe_exl3_kernels_load(C.byref(self.h)))

    @classmethod
    def load(cls):
        return cls()

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_exl3_kernels_destroy(self.h)
            self.h = None

    def set_option(self, name: str, value: int):
        """A switch of the launch paths ("fused_rot", "group", "hat_rows", ...: include/fe_exl3.h)."""
        check(_lib.lib().fe_exl3_kernels_set_option(self.h, name.encode(), int(value)))

    def reconstruct_hat_f16(self, view: Exl3View, out, stream=None):
        """Rotated-basis W_hat as fp16 [k][n] (gpu/mod.rs:159-165)."""
        v = view.c()
        check(_lib.lib().fe_exl3_reconstruct_hat_f16(self.h, _stream(stream), C.byref(v), out.data_ptr()))

    @staticmethod
    def recon_scratch_bytes(view: Exl3View):
        return view.k * view.n * 4  # gpu/mod.rs:104-108

    def reconstruct_bf16(self, view: Exl3View, out, layout, scratch, stream=None):
        """Original-basis W as bf16, layout "KN" or "NK" (gpu/mod.rs:110-157)."""
        v = view.c()
        check(_lib.lib().fe_exl3_reconstruct_bf16(self.h, _stream(stream), C.byref(v), out.data_ptr(), 0 if layout == "KN" else 1,
                                                  scratch.data_ptr(), scratch.numel() * scratch.element_size()))

    def probe_stream_read(self, buf, grid, launches, stream=None):
        ms = C.c_float()
        check(_lib.lib().fe_exl3_probe_stream_read(self.h, _stream(stream), buf.data_ptr(), buf.numel() * buf.element_size(), grid,
                                                   launches, C.byref(ms)))
        return ms.value

    PROBE_OPS = ("add", "and", "mul_lo", "mad_u24", "bfe", "alignbit", "perm", "sad_u8", "sad_hi_u8", "pk_fma_f16", "fma_f32", "dpp_mov")

    def probe_op(self, op, grid, iters, launches, stream=None):
        """Milliseconds per launch of grid x 256 lanes x 8 chains x iters dependent instructions `op` (PROBE_OPS)."""
        ms = C.c_float()
        check(_lib.lib().fe_exl3_probe_op(self.h, _stream(stream), op.encode(), grid, iters, launches, C.byref(ms)))
        return ms.value

    def probe_decode(self, bits, grid, iters, launches, stream=None):
        ms = C.c_float()
        check(_lib.lib().fe_exl3_probe_decode(self.h, _stream(stream), bits, grid, iters, launches, C.byref(ms)))
        return ms.value


def cu_count() -> int:
    _lib.init()
    n = C.c_int()
    check(_lib.lib().fe_hip_cu_count(C.byref(n)))
    return n.value


class Linear:
    """An EXL3 linear served straight from the trellis (crates/fe-exl3/src/linear.rs:163-342)."""

    def __init__(self, kern: Kernels, name: str, view: Exl3View, plan: Plan, owned=None):
        self.kern, self.name, self.view, self.owned = kern, name, view, owned
        self.h = C.c_void_p()
        v, p = view.c(), plan.c()
        check(_lib.lib().fe_exl3_linear_from_view(C.byref(self.h), kern.h, name.encode(), C.byref(v), C.byref(p)))
        self.k, self.n, self.bits, self.plan = view.k, view.n, view.bits, plan

    @staticmethod
    def plan_for(k, n, bits, blocks) -> Plan:
        p = PlanC()
        check(_lib.lib().fe_exl3_plan_for(k, n, bits, blocks, C.byref(p)))
        return Plan(p.sk, p.wk, p.ver, p.occ)

    @classmethod
    def new(cls, kern, w: DeviceExl3, blocks: int):
        return cls.with_plan(kern, w, cls.plan_for(w.view.k, w.view.n, w.view.bits, blocks))

    @classmethod
    def with_plan(cls, kern, w: DeviceExl3, plan: Plan):
        return cls(kern, w.name, w.view, plan, owned=w)

    @classmethod
    def from_view(cls, kern, name, view: Exl3View, plan: Plan):
        return cls(kern, name, view, plan)

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_exl3_linear_destroy(self.h)
            self.h = None

    def weight_bytes(self):
        return _lib.lib().fe_exl3_linear_weight_bytes(self.h)

    def forward(self, x, x_dtype: Dtype, y, y_dtype: Dtype, rows: int, ws: "Workspace", stream=None):
        """y[rows][n] = x[rows][k] @ W (linear.rs:273-287)."""
        check(_lib.lib().fe_exl3_linear_forward(self.h, self.kern.h, _stream(stream), x.data_ptr(), int(x_dtype), y.data_ptr(),
                                                int(y_dtype), rows, ws.h))

    def forward_static(self, x, x_dtype: Dtype, y, y_dtype: Dtype, rows: int, stream=None):
        """forward() without a Workspace and without any allocation: the scratch memory is a static device array of the
        library (1..16 rows; larger shapes than it holds raise FeError). Calls that overlap on one GPU race."""
        check(_lib.lib().fe_exl3_linear_forward_static(self.h, self.kern.h, _stream(stream), x.data_ptr(), int(x_dtype),
                                                       y.data_ptr(), int(y_dtype), rows))

    def forward_swiglu(self, gate, up, ld: int, y, y_dtype: Dtype, rows: int, ws: "Workspace", stream=None):
        """y[rows][n] = SwiGLU(gate, up)[rows][k] @ W with bf16 gate / up of row stride ld (pointers or tensors): the
        activation bf16(bf16(silu(gate)) * up) is formed as the input rotation reads it."""
        gp = gate if isinstance(gate, int) else gate.data_ptr()
        up_ = up if isinstance(up, int) else up.data_ptr()
        check(_lib.lib().fe_exl3_linear_forward_swiglu(self.h, self.kern.h, _stream(stream), gp, up_, ld, y.data_ptr(), int(y_dtype),
                                                       rows, ws.h))

    def keep_decoded(self, on: bool = True, stream=None):
        """Decode the trellis once into fp16 tiles kept with the linear (2 bytes a weight): calls with more than 64 rows
        then run the GEMM over them without decoding."""
        check(_lib.lib().fe_exl3_linear_keep_decoded(self.h, _stream(stream), int(on)))

    def decoded_w_hat(self):
        """The kept tiles un-swizzled: W_hat as fp16 bits [k][n] (host uint16 array), exactly the values the decoder of
        the hot loops produced (keep_decoded() first)."""
        ptr, nbytes = C.c_uint64(), C.c_size_t()
        check(_lib.lib().fe_exl3_linear_decoded(self.h, C.byref(ptr), C.byref(nbytes)))
        if not ptr.value:
            raise FeError(-1, "no decoded tiles: call keep_decoded() first")
        raw = np.empty(nbytes.value // 2, np.uint16)
        check(_lib.lib().fe_hip_synchronize())
        check(_lib.lib().fe_hip_memcpy_dtoh(raw.ctypes.data_as(C.c_void_p), ptr.value, nbytes.value))
        ktiles, tiles_n = self.k // 64, (self.n // 128 + 1) // 2
        blocks = raw.reshape(tiles_n, ktiles, 256, 8, 8)  # [tn][kt][column r][position][8 values]
        r = np.arange(256)[:, None]
        pos = np.arange(8)[None, :] ^ (r & 7) ^ ((r >> 3) & 1)  # where chunk c of column r lies
        chunks = np.take_along_axis(blocks, np.broadcast_to(pos[None, None, :, :, None], blocks.shape), axis=3)  # [tn][kt][r][c][8]
        w = chunks.reshape(tiles_n, ktiles, 256, 64).transpose(1, 3, 0, 2).reshape(self.k, tiles_n * 256)
        return np.ascontiguousarray(w[:, :self.n])

    def forward_is_one_launch(self, rows: int) -> bool:
        """Whether forward() with this many rows is the decode GEMV alone, rotating its own input."""
        return bool(_lib.lib().fe_exl3_linear_forward_is_one_launch(self.h, rows))

    def rotate_input(self, x, x_dtype: Dtype, rows: int, ws: "Workspace", stream=None):
        check(_lib.lib().fe_exl3_linear_rotate_input(self.h, self.kern.h, _stream(stream), x.data_ptr(), int(x_dtype), rows, ws.h))

    def gemv_rotated(self, xh, y, y_dtype: Dtype, rows: int, ws: "Workspace", stream=None):
        ptr = xh if isinstance(xh, int) else xh.data_ptr()
        check(_lib.lib().fe_exl3_linear_gemv_rotated(self.h, _stream(stream), ptr, y.data_ptr(), int(y_dtype), rows, ws.h))


def _group_handles(linears):
    return (C.c_void_p * len(linears))(*[l.h for l in linears])


def forward_group(linears, x, x_dtype: Dtype, ys, y_dtype: Dtype, rows: int, ws: "Workspace", stream=None):
    """ys[i][rows][n_i] = x[rows][k] @ W_i for linears of one input (q, k, v; gate, up): one GEMV launch for all of them
    (forward_group_launches: 1 or 2 with the rotation), else one forward per member; the same bits either way."""
    kern = linears[0].kern
    ptrs = (C.c_uint64 * len(ys))(*[y.data_ptr() for y in ys])
    check(_lib.lib().fe_exl3_linear_forward_group(_group_handles(linears), len(linears), kern.h, _stream(stream), x.data_ptr(),
                                                  int(x_dtype), ptrs, int(y_dtype), rows, ws.h))


def forward_group_launches(linears, rows: int, ws: "Workspace") -> int:
    """Launches of forward_group: 1 (the GEMV rotates its input), 2 (a rotation for all members, then the GEMV), 0 (the
    members run one after the other)."""
    return _lib.lib().fe_exl3_linear_forward_group_launches(_group_handles(linears), len(linears), rows, ws.h)


def mlp_forward(gate, up, down, x, x_dtype: Dtype, yg, yu, y, y_dtype: Dtype, rows: int, ws: "Workspace", stream=None):
    """The decode MLP block: yg = x @ W_gate, yu = x @ W_up (bf16), y (+)= SwiGLU(yg, yu) @ W_down; one launch where
    mlp_forward_launches says so, else the grouped gate + up launch followed by down's forward_swiglu (the same bits)."""
    check(_lib.lib().fe_exl3_mlp_forward(gate.h, up.h, down.h, gate.kern.h, _stream(stream), x.data_ptr(), int(x_dtype),
                                         yg.data_ptr(), yu.data_ptr(), y.data_ptr(), int(y_dtype), rows, ws.h))


def mlp_forward_launches(gate, up, down, rows: int, y_dtype: Dtype, ws: "Workspace") -> int:
    return _lib.lib().fe_exl3_mlp_forward_launches(gate.h, up.h, down.h, rows, int(y_dtype), ws.h)


class Workspace:
    """Scratch shared by every Linear on one stream (linear.rs:136-161)."""

    def chain_status(self) -> int:
        """Synchronizes and returns the error word of the one-launch MLP (0: all its bounded waits were met); clears it."""
        e = C.c_uint32()
        check(_lib.lib().fe_exl3_workspace_chain_status(self.h, C.byref(e)))
        return e.value

    def __init__(self, linears, max_rows: int):
        _lib.init()
        self.h = C.c_void_p()
        arr = (C.c_void_p * max(len(linears), 1))(*[l.h for l in linears])
        check(_lib.lib().fe_exl3_workspace_create(C.byref(self.h), arr, len(linears), max_rows))
        xh, mr, mk = C.c_uint64(), C.c_uint32(), C.c_uint32()
        check(_lib.lib().fe_exl3_workspace_xh(self.h, C.byref(xh), C.byref(mr), C.byref(mk)))
        self.xh_ptr, self.max_rows, self.max_k = xh.value, mr.value, mk.value

    def xh(self, rows, k):
        """The first rows x k rotated inputs as a host uint16 array (fp16 bits)."""
        out = np.empty((rows, k), np.uint16)
        for r in range(rows):
            check(_lib.lib().fe_hip_memcpy_dtoh(out[r].ctypes.data_as(C.c_void_p), self.xh_ptr + 2 * r * k, 2 * k))
        return out

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None and _lib._lib is not None:
            _lib._lib.fe_exl3_workspace_destroy(self.h)
            self.h = None


def _graph_us(fn, inner: int, reps: int = 5, ramp_ms: float = 40.0) -> float:
    """Microseconds per call of fn(stream) with `inner` calls captured into one HIP graph and the graph replayed: the
    launches run back to back as they do under a captured decode step, with no host time between them. The graph is first
    replayed untimed for `ramp_ms`: after host work the GPU needs about 30 ms of launches to reach the clocks it holds in a
    decode loop, and until then every launch reads 7-13 % slow."""
    lib = _lib.lib()
    s, a, b, g = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(lib.fe_hip_stream_create(C.byref(s)))
    check(lib.fe_hip_event_create(C.byref(a)))
    check(lib.fe_hip_event_create(C.byref(b)))
    try:
        fn(s)
        check(lib.fe_hip_stream_sync(s))
        check(lib.fe_hip_graph_begin(s))
        for _ in range(inner):
            fn(s)
        check(lib.fe_hip_graph_end(s, C.byref(g)))
        ms = C.c_float()
        check(lib.fe_hip_event_record(a, s))
        check(lib.fe_hip_graph_launch(g, s))
        check(lib.fe_hip_event_record(b, s))
        check(lib.fe_hip_event_sync(b))
        check(lib.fe_hip_event_elapsed_ms(C.byref(ms), a, b))
        for _ in range(int(ramp_ms / max(ms.value, 1e-3))):
            check(lib.fe_hip_graph_launch(g, s))
        best = float("inf")
        for _ in range(3):
            check(lib.fe_hip_event_record(a, s))
            for _ in range(reps):
                check(lib.fe_hip_graph_launch(g, s))
            check(lib.fe_hip_event_record(b, s))
            check(lib.fe_hip_event_sync(b))
            check(lib.fe_hip_event_elapsed_ms(C.byref(ms), a, b))
            best = min(best, ms.value * 1e3 / (reps * inner))
        check(lib.fe_hip_graph_destroy(g))
        return best
    finally:
        lib.fe_hip_event_destroy(a)
        lib.fe_hip_event_destroy(b)
        lib.fe_hip_stream_destroy(s)


def tune(kern: Kernels, t: Exl3Tensor, iters: int = 5, w16: float = 0.25, copies_bytes: int = 600 << 20,
         occs=(2, 3, 4, 5), min_units=(2, 4, 8)):
    """Times every candidate plan on one tensor shape at 1 and 16 rows and returns (best plan, table), the table a list of
    (plan, us at 1 row, us at 16 rows) sorted by us1 + w16 * us16 (the measure of
    crates/fe-exl3/src/bin/exl3-tune.rs:75-118). Launches cycle over enough copies of the weights that none is served
    from a cache and are replayed from a graph, `iters` replays of two passes over the copies. Candidates: occ programs
    per CU, each a run of at least wk units of 128 channels x 128 columns; plans that come to the same program count are
    timed once."""
    import torch
    copies = max(2, min(64, copies_bytes // max(1, t.trellis_bytes()) + 1))
    devs = [DeviceExl3.upload_strips(t) for _ in range(copies)]
    x = torch.full((16, t.k), 1.0, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((16, t.n), dtype=torch.bfloat16, device="cuda")
    units, cus = (t.k // 128) * (t.n // 128), cu_count()
    table, seen = [], set()
    for occ in occs:
        for wk in min_units:
            programs = max(1, min(occ * cus, units // wk))
            if (occ, programs) in seen:
                continue
            seen.add((occ, programs))
            p = Plan(-(-programs // (t.n // 128)), wk, 3, occ)
            lins = [Linear.from_view(kern, d.name, d.view, p) for d in devs]
            ws = Workspace(lins[:1], 16)
            us = []
            for rows in (1, 16):
                at = [0]

                def fn(s):
                    lins[at[0] % copies].forward(x, Dtype.Bf16, y, Dtype.Bf16, rows, ws, stream=s)
                    at[0] += 1
                us.append(_graph_us(fn, 2 * copies, iters))
            table.append((p, us[0], us[1]))
    table.sort(key=lambda e: e[1] + w16 * e[2])
    return table[0][0], table


if __name__ == "__main__":
    # python -m ferrite_amd.exl3 tune [k n bits]...: prints rows for ferrite_amd/csrc/fe_exl3_plans.h
    import sys
    from . import synth
    if len(sys.argv) >= 2 and sys.argv[1] == "tune":
        shapes = [tuple(int(v) for v in a.split("x")) for a in sys.argv[2:]] or [
            (k, n, b) for b in (3, 4, 5) for k, n in ((5120, 17408), (17408, 5120))] + [(5120, 5120, 4), (5120, 1024, 4)]
        kern = Kernels.load()
        for k, n, bits in shapes:
            best, table = tune(kern, synth.exl3_tensor(k, n, bits, 1))
            print(f"    {{{k}, {n}, {bits}, {cu_count()}, {best.occ}, {best.wk}}},  // " +
                  "; ".join(f"occ {p.occ} wk {p.wk}: {u1:.1f} / {u16:.1f} us" for p, u1, u16 in table[:4]), flush=True)
