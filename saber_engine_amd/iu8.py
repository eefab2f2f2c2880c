"""Python binding of the C ABI in include/saber_iu8.h (ctypes; no compute happens here).

The names mirror the reference's host interface for this path: `resolve(WKind, m, n, k)`
(crates/saber-kernels/src/macaq_iu8.rs:425), `PluginSet.load_dir` (crates/saber-exec/src/
loader.rs:318), `Launcher.launch_op` (crates/saber-exec/src/launch.rs:590).  Device memory and
streams are the caller's (torch tensors' data_ptr() / torch.cuda streams in the tests).

The library has no CPU fallback: opening a context without a GPU, or before the code objects
were built, raises.
"""
import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
LIB_PATH = os.path.join(PKG, "libsaber_iu8.so")
PREBUILT = os.path.join(ROOT, "prebuilt", "gfx950")
# the parity suite's test-only object (accumulator and table taps), outside the plugin directory
TAPS_MANIFEST = os.path.join(PREBUILT, "taps", "iu8_taps.manifest.toml")
BAND_TABLE = os.path.join(PREBUILT, "macaq_iu8.band.toml")
DEVICE_PROFILE = os.path.join(PREBUILT, "device_profile.toml")

W4, W8 = 0, 1
ARG_BUFFER, ARG_NULL_BUFFER, ARG_I32, ARG_F32, ARG_I64 = 0, 1, 2, 3, 4
WS_SCRATCH, WS_PERSISTENT = 0, 1
E_RULE, E_PARSE, E_VALIDATE, E_HIP, E_ARG, E_IO, E_NOTLOADED = -1, -2, -3, -4, -5, -6, -7
REFUSED_KERNARG, REFUSED_WAVE, REFUSED_METADATA = 1, 2, 3


class Slot(C.Structure):
    _fields_ = [("name", C.c_char * 24), ("offset", C.c_uint32), ("size", C.c_uint32), ("kind", C.c_uint32),
                ("ival", C.c_int64), ("fval", C.c_float)]


class Workspace(C.Structure):
    _fields_ = [("name", C.c_char * 24), ("kind", C.c_uint32), ("bytes", C.c_uint64), ("zero_once", C.c_uint32)]


class Desc(C.Structure):
    _fields_ = [("op", C.c_char * 24), ("plugin", C.c_char * 24), ("kernel", C.c_char * 64), ("grid", C.c_uint32 * 3),
                ("block", C.c_uint32 * 3), ("shared_bytes", C.c_uint32), ("kernarg_bytes", C.c_uint32),
                ("n_args", C.c_uint32), ("args", Slot * 24), ("n_workspaces", C.c_uint32), ("workspaces", Workspace * 4),
                ("n_launches", C.c_uint32), ("ks", C.c_uint32)]

    def summary(self):
        g, b = self.grid, self.block
        return f"{self.kernel.decode()} grid={g[0]}x{g[1]}x{g[2]} block={b[0]} n_launches={self.n_launches}"

    def arg(self, name):
        for i in range(self.n_args):
            if self.args[i].name.decode() == name:
                return self.args[i]
        return None

    def workspace(self, name):
        for i in range(self.n_workspaces):
            if self.workspaces[i].name.decode() == name:
                return self.workspaces[i]
        return None


class Binding(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ptr", C.c_void_p)]


class Counters(C.Structure):
    _fields_ = [("plugins_loaded", C.c_uint32), ("kernels_loaded", C.c_uint32), ("refused_kernarg", C.c_uint32),
                ("refused_wave", C.c_uint32), ("refused_metadata", C.c_uint32), ("launches", C.c_uint32)]


MOE_TABLE_FIELDS = ("topk_ids", "topk_w", "route_pos", "row_tok", "row_route", "tile_expert", "tile_row0", "tile_rows",
                    "expert_cnt", "meta", "blk_cnt", "rank", "arrive", "silu_lut", "sgate")


class MoeTables(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in MOE_TABLE_FIELDS]


class IU8Error(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"[{code}] {msg}")
        self.code = code


_lib = None


def lib():
    """The loaded C library. Raises if it was not built (run __graft_entry__.build())."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise IU8Error(E_NOTLOADED, f"{LIB_PATH} is not built; run `python -m saber_engine_amd.kbuild`")
        try:  # share the process's HIP runtime with torch when torch is in use
            import torch  # noqa: F401
        except Exception:
            pass
        L = C.CDLL(LIB_PATH)
        L.saber_iu8_last_error.restype = C.c_char_p
        L.saber_iu8_a_bytes.restype = C.c_size_t
        L.saber_iu8_a_bytes.argtypes = [C.c_uint32, C.c_uint32]
        L.saber_iu8_a_offset.restype = C.c_uint64
        L.saber_iu8_a_offset.argtypes = [C.c_uint32] * 3
        L.saber_iu8_w4_offset.restype = C.c_uint64
        L.saber_iu8_w4_offset.argtypes = [C.c_uint32] * 3 + [C.POINTER(C.c_uint32)]
        L.saber_iu8_open.argtypes = [C.c_char_p, C.c_int, C.POINTER(C.c_void_p)]
        L.saber_iu8_close.argtypes = [C.c_void_p]
        L.saber_iu8_launch.argtypes = [C.c_void_p, C.POINTER(Desc), C.POINTER(Binding), C.c_uint32, C.c_void_p]
        L.saber_iu8_quant.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
        L.saber_iu8_quant_rowmajor.argtypes = L.saber_iu8_quant.argtypes
        L.saber_iu8_gemm.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 5 + [C.c_uint32] * 3 + [C.c_void_p] * 3
        L.saber_iu8_rowscale.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
        L.saber_iu8_linear_prefill_fused.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 5 + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_gemm_static.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 5 + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_static_workspace_reset.argtypes = [C.c_void_p, C.c_void_p]
        L.saber_iu8_static_workspace_bytes.restype = C.c_uint64
        L.saber_iu8_gemm_acc.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 3 + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_fused_holds.argtypes = [C.c_uint32, C.c_uint32]
        L.saber_iu8_mlp_chain_holds.argtypes = [C.c_uint32] * 3
        L.saber_iu8_mlp_chain_pays.argtypes = [C.c_uint32] * 3
        L.saber_iu8_gate_up_act_holds.argtypes = [C.c_uint32] * 3
        L.saber_iu8_resolve_gate_up_act.argtypes = [C.c_uint32] * 3 + [C.POINTER(Desc)]
        L.saber_iu8_gate_up_act.argtypes = [C.c_void_p] * 7 + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_pair.argtypes = [C.POINTER(Desc)] * 3
        L.saber_iu8_pair_ordered.argtypes = [C.POINTER(Desc)] * 2 + [C.c_int, C.POINTER(Desc)]
        L.saber_iu8_load_plugin.argtypes = [C.c_void_p, C.c_char_p]
        L.saber_iu8_band_toml.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
        L.saber_iu8_device_profile_toml.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
        L.saber_iu8_gemm_pair.argtypes = [C.c_void_p] * 6 + [C.c_uint32] + [C.c_void_p] * 3 + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_linear_fused.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 6 + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_resolve_mlp_chain.argtypes = [C.c_uint32] * 4 + [C.c_void_p]
        L.saber_iu8_mlp_chain.argtypes = [C.c_void_p] * 10 + [C.c_uint32] * 4 + [C.c_void_p]
        L.saber_iu8_quant_had.argtypes = [C.c_void_p] * 4 + [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        L.saber_iu8_silu_mul_quant_had.argtypes = [C.c_void_p] * 4 + [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        L.saber_iu8_silu_mul_quant_had_lut.argtypes = [C.c_void_p] * 4 + [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]
        L.saber_iu8_add_rms_quant_had.argtypes = [C.c_void_p] * 7 + [C.c_uint32, C.c_uint32, C.c_float, C.c_void_p, C.c_void_p]
        L.saber_iu8_gdn_norm_quant_had.argtypes = [C.c_void_p] * 3 + [C.c_int64] + [C.c_void_p] * 3 + [
            C.c_uint32, C.c_uint32, C.c_float, C.c_void_p, C.c_void_p]
        L.saber_iu8_attn_gate_quant_had.argtypes = [C.c_void_p] * 5 + [C.c_uint32] * 4 + [C.c_void_p, C.c_void_p]
        L.saber_iu8_attn_gate_quant_had_lut.argtypes = [C.c_void_p] * 5 + [C.c_uint32] * 4 + [C.c_void_p, C.c_void_p, C.c_void_p]
        L.saber_iu8_sigmoid_table.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.saber_iu8_get_counters.argtypes = [C.c_void_p, C.POINTER(Counters)]
        L.saber_iu8_has_kernel.argtypes = [C.c_void_p, C.c_char_p]
        for fn in ("saber_iu8_moe_rows_cap", "saber_iu8_moe_rows_cap_shared", "saber_iu8_moe_tile_blocks"):
            getattr(L, fn).restype = C.c_uint32
            getattr(L, fn).argtypes = [C.c_uint32] * 3
        for fn in ("saber_iu8_moe_tiles_cap", "saber_iu8_moe_tiles_cap_shared"):
            getattr(L, fn).restype = C.c_uint32
            getattr(L, fn).argtypes = [C.c_uint32] * 4
        L.saber_iu8_moe_route.argtypes = [C.c_void_p, C.c_void_p] + [C.c_uint32] * 4 + [C.POINTER(MoeTables), C.c_void_p]
        L.saber_iu8_moe_route_quant.argtypes = [C.c_void_p] * 5 + [C.c_uint32] * 5 + [C.POINTER(MoeTables), C.c_void_p]
        L.saber_iu8_moe_grouped.argtypes = ([C.c_void_p] * 5 + [C.c_uint32, C.c_uint32, C.c_int] + [C.c_uint32] * 4 +
                                            [C.POINTER(MoeTables), C.c_void_p])
        L.saber_iu8_moe_quant_rows.argtypes = [C.c_void_p] * 4 + [C.c_uint32, C.c_uint32, C.POINTER(MoeTables), C.c_void_p]
        L.saber_iu8_moe_back_holds.restype = C.c_int
        L.saber_iu8_moe_back_holds.argtypes = [C.c_uint32, C.c_uint32]
        L.saber_iu8_moe_back_pays.restype = C.c_int
        L.saber_iu8_moe_back_pays.argtypes = [C.c_uint32] * 5
        L.saber_iu8_moe_gate_up_act.argtypes = [C.c_void_p] * 5 + [C.c_uint32] * 6 + [C.POINTER(MoeTables), C.c_void_p]
        L.saber_iu8_moe_down_rows.argtypes = [C.c_void_p] * 4 + [C.c_uint32] * 6 + [C.POINTER(MoeTables), C.c_void_p]
        L.saber_iu8_moe_silu_mul_quant.argtypes = [C.c_void_p] * 4 + [C.c_uint32, C.c_uint32, C.POINTER(MoeTables), C.c_void_p]
        L.saber_iu8_moe_combine.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(MoeTables), C.c_void_p] + [C.c_uint32] * 3 + [C.c_void_p]
        L.saber_iu8_silu_table.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise IU8Error(rc, lib().saber_iu8_last_error().decode())


# ---------------------------------------------------------------------------- launch law (host)

def resolve(wkind, m, n, k):
    d = Desc()
    _check(lib().saber_iu8_resolve(wkind, m, n, k, C.byref(d)))
    return d


def describe(kernel, m, n, k, ks=1):
    d = Desc()
    _check(lib().saber_iu8_describe(kernel.encode(), m, n, k, ks, C.byref(d)))
    return d


def pair(first, second):
    """Two W4 decode descriptors of one M, K -> the one-dispatch pair (macaq_iu8.rs:632-704)."""
    d = Desc()
    _check(lib().saber_iu8_pair(C.byref(first), C.byref(second), C.byref(d)))
    return d


def pair_ordered(first, second, second_first):
    """The pair with its block order named: the second problem's workgroups first (`pairb`) or last."""
    d = Desc()
    _check(lib().saber_iu8_pair_ordered(C.byref(first), C.byref(second), int(bool(second_first)), C.byref(d)))
    return d


def band_toml():
    """The launch law as TOML text (what the build step writes to BAND_TABLE)."""
    need = C.c_size_t(0)
    lib().saber_iu8_band_toml(None, 0, C.byref(need))
    buf = C.create_string_buffer(need.value)
    _check(lib().saber_iu8_band_toml(buf, need.value, None))
    return buf.value.decode()


def device_profile_toml():
    """The target's DeviceProfile as TOML text (what the build step writes to DEVICE_PROFILE)."""
    need = C.c_size_t(0)
    lib().saber_iu8_device_profile_toml(None, 0, C.byref(need))
    buf = C.create_string_buffer(need.value)
    _check(lib().saber_iu8_device_profile_toml(buf, need.value, None))
    return buf.value.decode()


def fused_holds(m, k):
    return bool(lib().saber_iu8_fused_holds(m, k))


def fused_small_holds(m, k):
    """Up to 4 rows whose codes fit 20 KiB: the `_tm1` fused kernel."""
    mr = 1
    while mr < m:
        mr *= 2
    return 1 <= m <= 4 and mr * k <= 20 * 1024


def mlp_chain_holds(m, hidden, inter):
    return bool(lib().saber_iu8_mlp_chain_holds(m, hidden, inter))


def gate_up_act_holds(m, hidden, inter):
    return bool(lib().saber_iu8_gate_up_act_holds(m, hidden, inter))


def resolve_gate_up_act(m, hidden, inter):
    d = Desc()
    _check(lib().saber_iu8_resolve_gate_up_act(m, hidden, inter, C.byref(d)))
    return d


def mlp_chain_pays(m, hidden, inter):
    """The one-launch MLP measured faster than the three launches at this shape."""
    return bool(lib().saber_iu8_mlp_chain_pays(m, hidden, inter))


def resolve_fused(wkind, m, n, k):
    d = Desc()
    _check(lib().saber_iu8_resolve_fused(wkind, m, n, k, C.byref(d)))
    return d


MLP_CHAIN_STATE_BYTES = 13 * 1024
MLP_CHAIN_STATUS_OFFSET = 12 * 1024


def resolve_mlp_chain(m, hidden, inter, spin=0):
    d = Desc()
    _check(lib().saber_iu8_resolve_mlp_chain(m, hidden, inter, spin, C.byref(d)))
    return d


def resolve_prefill_fused(wkind, m, n, k):
    d = Desc()
    _check(lib().saber_iu8_resolve_prefill_fused(wkind, m, n, k, C.byref(d)))
    return d


def resolve_quant(m, k):
    d = Desc()
    _check(lib().saber_iu8_resolve_quant(m, k, C.byref(d)))
    return d


def resolve_silu_mul_quant(rows, n):
    d = Desc()
    _check(lib().saber_iu8_resolve_silu_mul_quant(rows, n, C.byref(d)))
    return d


def describe_raw(kernel, grid, block, plugin="", **scalars):
    """Descriptor for any loaded kernel with an explicit launch shape; scalars set by name."""
    d = Desc()
    g = (C.c_uint32 * 3)(*grid)
    _check(lib().saber_iu8_describe_raw(kernel.encode(), plugin.encode(), g, block, C.byref(d)))
    for name, v in scalars.items():
        _check(lib().saber_iu8_desc_set_i32(C.byref(d), name.encode(), C.c_int64(int(v))))
    return d


def signature(kernel):
    slots = (Slot * 24)()
    n, b = C.c_uint32(), C.c_uint32()
    _check(lib().saber_iu8_signature(kernel.encode(), slots, 24, C.byref(n), C.byref(b)))
    return [(slots[i].name.decode(), slots[i].offset, slots[i].size, slots[i].kind) for i in range(n.value)], b.value


def _bindings(bufs):
    arr = (Binding * max(1, len(bufs)))()
    for i, (name, ptr) in enumerate(bufs.items()):
        arr[i].name = name.encode()
        arr[i].ptr = ptr
    return arr


def pack_kernarg(desc, bufs):
    """bufs: {name: device address}. Returns the kernarg image as bytes."""
    img = (C.c_uint8 * 256)()
    n = C.c_uint32()
    _check(lib().saber_iu8_pack_kernarg(C.byref(desc), _bindings(bufs), len(bufs), img, 256, C.byref(n)))
    return bytes(img[:n.value])


# ---------------------------------------------------------------------------- layouts (host)

def a_bytes(m, k):
    return lib().saber_iu8_a_bytes(m, k)


def repack_w4(canonical):
    c = np.ascontiguousarray(canonical, dtype=np.uint8)
    n, k = c.shape[0], c.shape[1] * 2
    out = np.empty(n * k // 2, np.uint8)
    _check(lib().saber_iu8_repack_w4(c.ctypes.data_as(C.c_void_p), n, k, out.ctypes.data_as(C.c_void_p)))
    return out


def repack_w8(rowmajor):
    w = np.ascontiguousarray(rowmajor, dtype=np.int8)
    n, k = w.shape
    out = np.empty(n * k, np.uint8)
    _check(lib().saber_iu8_repack_w8(w.ctypes.data_as(C.c_void_p), n, k, out.ctypes.data_as(C.c_void_p)))
    return out


def repack_weights(W, w8):
    return repack_w8(W) if w8 else repack_w4(W)


def repack_a(rowmajor):
    a = np.ascontiguousarray(rowmajor, dtype=np.int8)
    m, k = a.shape
    out = np.empty(a_bytes(m, k), np.uint8)
    _check(lib().saber_iu8_repack_a(a.ctypes.data_as(C.c_void_p), m, k, out.ctypes.data_as(C.c_void_p)))
    return out


def unpack_a(frag, m, k):
    f = np.ascontiguousarray(frag, dtype=np.uint8)
    out = np.empty((m, k), np.int8)
    _check(lib().saber_iu8_unpack_a(f.ctypes.data_as(C.c_void_p), m, k, out.ctypes.data_as(C.c_void_p)))
    return out


# ---------------------------------------------------------------------------- manifests (host)

def manifest_validate(path, arch="gfx950"):
    """Returns (rc, refusal, message)."""
    refusal = C.c_int(0)
    rc = lib().saber_iu8_manifest_validate(path.encode(), arch.encode() if arch else None, C.byref(refusal))
    return rc, refusal.value, lib().saber_iu8_last_error().decode() if rc else ""


# ---------------------------------------------------------------------------- device side

class Context:
    """A loaded plugin set on one device (PluginSet + Launcher)."""

    def __init__(self, prebuilt_dir=PREBUILT, device=0):
        self._h = C.c_void_p()
        _check(lib().saber_iu8_open(prebuilt_dir.encode(), device, C.byref(self._h)))

    def close(self):
        if self._h:
            lib().saber_iu8_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load_plugin(self, manifest_path):
        """Add one plugin from outside the plugin directory (the parity suite's taps)."""
        _check(lib().saber_iu8_load_plugin(self._h, manifest_path.encode()))

    def load_taps(self):
        self.load_plugin(TAPS_MANIFEST)

    def counters(self):
        c = Counters()
        _check(lib().saber_iu8_get_counters(self._h, C.byref(c)))
        return c

    def has_kernel(self, name):
        return bool(lib().saber_iu8_has_kernel(self._h, name.encode()))

    def launch(self, desc, bufs, stream=0):
        _check(lib().saber_iu8_launch(self._h, C.byref(desc), _bindings(bufs), len(bufs), stream))

    def quant(self, x, q, scale, m, k, stream=0):
        _check(lib().saber_iu8_quant(self._h, x, q, scale, m, k, stream))

    def quant_rowmajor(self, x, q, scale, m, k, stream=0):
        _check(lib().saber_iu8_quant_rowmajor(self._h, x, q, scale, m, k, stream))

    def gemm(self, wkind, a, a_scale, w, w_scale, c, m, n, k, partial=None, counter=None, stream=0):
        _check(lib().saber_iu8_gemm(self._h, wkind, a, a_scale, w, w_scale, c, m, n, k, partial, counter, stream))

    def gate_up_act(self, a, a_scale, w_gu, ws_gu, gu, p, m, hidden, inter, stream=0):
        _check(lib().saber_iu8_gate_up_act(self._h, a, a_scale, w_gu, ws_gu, gu, p, m, hidden, inter, stream))

    def rowscale(self, x, scale, m, k, stream=0):
        _check(lib().saber_iu8_rowscale(self._h, x, scale, m, k, stream))

    def linear_prefill_fused(self, wkind, x, a_scale, w, w_scale, c, m, n, k, stream=0):
        _check(lib().saber_iu8_linear_prefill_fused(self._h, wkind, x, a_scale, w, w_scale, c, m, n, k, stream))

    def gemm_static(self, wkind, a, a_scale, w, w_scale, c, m, n, k, stream=0):
        """gemm() with the split-K workspaces in the library's static device array: allocates nothing."""
        _check(lib().saber_iu8_gemm_static(self._h, wkind, a, a_scale, w, w_scale, c, m, n, k, stream))

    def static_workspace_reset(self, stream=0):
        """The static array's arrival counters back to zero (a fill kernel on `stream`): recovery after a split
        launch that was cut short."""
        _check(lib().saber_iu8_static_workspace_reset(self._h, stream))

    def gemm_pair(self, a, a_scale, w, w_scale, c, n, w_b, w_scale_b, c_b, n_b, m, k, stream=0):
        _check(lib().saber_iu8_gemm_pair(self._h, a, a_scale, w, w_scale, c, n, w_b, w_scale_b, c_b, n_b, m, k, stream))

    def linear_fused(self, wkind, x, w, w_scale, c, m, n, k, q=None, scale=None, stream=0):
        _check(lib().saber_iu8_linear_fused(self._h, wkind, x, w, w_scale, c, q, scale, m, n, k, stream))

    def mlp_chain(self, x, w_gu, ws_gu, w_dn, ws_dn, gu, p, state, c, m, hidden, inter, spin=0, stream=0):
        """gate+up -> SiLU * up + requant -> down in one persistent launch; `state` (MLP_CHAIN_STATE_BYTES)
        zero before the first use. A non-zero word at state + MLP_CHAIN_STATUS_OFFSET after the launch:
        a meeting timed out, c is undefined."""
        _check(lib().saber_iu8_mlp_chain(self._h, x, w_gu, ws_gu, w_dn, ws_dn, gu, p, state, c, m, hidden, inter, spin, stream))

    def quant_had(self, x, q, scale, m, k, had_t, stream=0):
        _check(lib().saber_iu8_quant_had(self._h, x, q, scale, m, k, had_t, stream))

    def silu_mul_quant_had(self, gu, q, scale, m, n, had_t, stream=0):
        _check(lib().saber_iu8_silu_mul_quant_had(self._h, gu, q, scale, m, n, had_t, stream))

    def silu_mul_quant_had_lut(self, gu, q, scale, m, n, had_t, silu_lut, stream=0):
        _check(lib().saber_iu8_silu_mul_quant_had_lut(self._h, gu, q, scale, m, n, had_t, silu_lut, stream))

    def add_rms_quant_had(self, y, res, w, q, scale, res_out, m, k, eps, had_t, stream=0):
        _check(lib().saber_iu8_add_rms_quant_had(self._h, y, res, w, q, scale, res_out, m, k, eps, had_t, stream))

    def gdn_norm_quant_had(self, x, z, z_stride, w, q, scale, m, n, eps, had_t, stream=0):
        _check(lib().saber_iu8_gdn_norm_quant_had(self._h, x, z, z_stride, w, q, scale, m, n, eps, had_t, stream))

    def attn_gate_quant_had(self, core, gate, q, scale, m, n, head_dim, gate_stride, had_t, stream=0):
        _check(lib().saber_iu8_attn_gate_quant_had(self._h, core, gate, q, scale, m, n, head_dim, gate_stride, had_t, stream))

    def attn_gate_quant_had_lut(self, core, gate, q, scale, m, n, head_dim, gate_stride, had_t, sigmoid_lut, stream=0):
        _check(lib().saber_iu8_attn_gate_quant_had_lut(self._h, core, gate, q, scale, m, n, head_dim, gate_stride, had_t, sigmoid_lut, stream))

    def sigmoid_table(self, out, stream=0):
        _check(lib().saber_iu8_sigmoid_table(self._h, out, stream))

    def gemm_acc(self, wkind, a, w, acc, m, n, k, stream=0):
        _check(lib().saber_iu8_gemm_acc(self._h, wkind, a, w, acc, m, n, k, stream))


    # ---- routed experts
    def moe_route(self, logits, tokens, experts, topk, tile_blocks, tables, stream=0):
        _check(lib().saber_iu8_moe_route(self._h, logits, tokens, experts, topk, tile_blocks, C.byref(tables), stream))

    def moe_route_quant(self, logits, x, q, scale, tokens, experts, topk, k, tile_blocks, tables, stream=0):
        _check(lib().saber_iu8_moe_route_quant(self._h, logits, x, q, scale, tokens, experts, topk, k, tile_blocks,
                                               C.byref(tables), stream))

    def moe_grouped(self, a, a_scale, xptr, c, n, k, gather, tokens, experts, topk, tile_blocks, tables, stream=0):
        _check(lib().saber_iu8_moe_grouped(self._h, a, a_scale, xptr, c, n, k, int(gather), tokens, experts, topk,
                                           tile_blocks, C.byref(tables), stream))

    def moe_gate_up_act(self, a, a_scale, xptr, p, inter, k, tokens, experts, topk, tile_blocks, tables, stream=0):
        _check(lib().saber_iu8_moe_gate_up_act(self._h, a, a_scale, xptr, p, inter, k, tokens, experts, topk, tile_blocks,
                                               C.byref(tables), stream))

    def moe_down_rows(self, p, xptr, y, n, inter, tokens, experts, topk, tile_blocks, tables, stream=0):
        _check(lib().saber_iu8_moe_down_rows(self._h, p, xptr, y, n, inter, tokens, experts, topk, tile_blocks,
                                             C.byref(tables), stream))

    def moe_quant_rows(self, x, q, scale, k, rows_cap, tables, stream=0):
        _check(lib().saber_iu8_moe_quant_rows(self._h, x, q, scale, k, rows_cap, C.byref(tables), stream))

    def moe_silu_mul_quant(self, gu, q, scale, n, rows_cap, tables, stream=0):
        _check(lib().saber_iu8_moe_silu_mul_quant(self._h, gu, q, scale, n, rows_cap, C.byref(tables), stream))

    def moe_combine(self, y, tables, out, tokens, topk, h, stream=0):
        _check(lib().saber_iu8_moe_combine(self._h, y, C.byref(tables), out, tokens, topk, h, stream))

    def silu_table(self, out, stream=0):
        _check(lib().saber_iu8_silu_table(self._h, out, stream))


def moe_rows_cap(tokens, topk, experts, shared=False):
    return (lib().saber_iu8_moe_rows_cap_shared if shared else lib().saber_iu8_moe_rows_cap)(tokens, topk, experts)


def moe_tiles_cap(tokens, topk, experts, tile_blocks, shared=False):
    return (lib().saber_iu8_moe_tiles_cap_shared if shared else lib().saber_iu8_moe_tiles_cap)(tokens, topk, experts, tile_blocks)


def moe_tile_blocks(tokens, topk, experts):
    return lib().saber_iu8_moe_tile_blocks(tokens, topk, experts)


def moe_back_pays(tokens, topk, experts, tile_blocks, inter):
    """The launch law's pick between the two-launch back half and the three launches."""
    return bool(lib().saber_iu8_moe_back_pays(tokens, topk, experts, tile_blocks, inter))


def moe_back_holds(tile_blocks, inter):
    """The routed back half as two launches (activation in gate+up's epilogue, requantisation in front of down's K loop)."""
    return bool(lib().saber_iu8_moe_back_holds(tile_blocks, inter))


def gemm_workspace(wkind, m, n, k):
    p, c = C.c_uint64(), C.c_uint64()
    _check(lib().saber_iu8_gemm_workspace(wkind, m, n, k, C.byref(p), C.byref(c)))
    return p.value, c.value
