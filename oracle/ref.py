"""TEST INFRASTRUCTURE: ctypes binding of the CPU oracle (oracle/w4a8_ref.c).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module; nothing under the product package does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libw4a8_ref.so")


def build(force=False):
    """Compile the oracle with gcc (idempotent unless force)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "w4a8_ref.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"] + ([] if force else []))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        L = _lib
        L.w4a8_bf16_rne.restype = C.c_uint16
        L.w4a8_bf16_rne.argtypes = [C.c_float]
        L.w4a8_bf16_f32.restype = C.c_float
        L.w4a8_bf16_f32.argtypes = [C.c_uint16]
        L.w4a8_epilogue.restype = C.c_uint16
        L.w4a8_epilogue.argtypes = [C.c_int32, C.c_float, C.c_float, C.c_int]
        L.w4a8_exp_nonpos.restype = C.c_float
        L.w4a8_exp_nonpos.argtypes = [C.c_float]
        L.w4a8_sigmoid.restype = C.c_float
        L.w4a8_sigmoid.argtypes = [C.c_float]
        L.w4a8_silu_bf16.restype = C.c_uint16
        L.w4a8_silu_bf16.argtypes = [C.c_uint16]
        L.w4a8_a_tiled_gfx12.restype = C.c_uint64
        L.w4a8_a_tiled_gfx12.argtypes = [C.c_uint32] * 3
        L.w4a8_w4_frag_gfx12.restype = C.c_uint64
        L.w4a8_w4_frag_gfx12.argtypes = [C.c_uint32] * 3 + [C.POINTER(C.c_uint32)]
        L.w4a8_rows_cap.restype = C.c_uint32
        L.w4a8_rows_cap.argtypes = [C.c_uint32] * 3
        L.w4a8_tiles_cap.restype = C.c_uint32
        L.w4a8_tiles_cap.argtypes = [C.c_uint32] * 4
        L.w4a8_isa.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def bf16_rne(x):
    """f32 array -> bf16 bits (uint16), round to nearest even."""
    x = _c(x, np.float32)
    L = lib()
    return np.array([L.w4a8_bf16_rne(float(v)) for v in x.ravel()], dtype=np.uint16).reshape(x.shape)


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def quant_bf16(x_bits):
    """bf16 bits [M,K] -> (int8 codes [M,K] row-major, f32 scale [M])."""
    x = _c(x_bits, np.uint16)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    s = np.empty(M, np.float32)
    lib().w4a8_quant_bf16(_p(x), C.c_int(M), C.c_int(K), _p(q), _p(s))
    return q, s


def quant_row_f32(x):
    x = _c(x, np.float32)
    q = np.empty(x.shape[0], np.int8)
    s = np.empty(1, np.float32)
    lib().w4a8_quant_row(_p(x), C.c_int(x.shape[0]), _p(q), _p(s))
    return q, s[0]


def gemm_ref(A, W, w8):
    """Scalar law. A int8 [M,K]; W uint8 canonical nibbles [N,K/2] (w8=0) or int8 [N,K]."""
    A = _c(A, np.int8)
    M, K = A.shape
    N = W.shape[0]
    S = np.empty((M, N), np.int32)
    if w8:
        W = _c(W, np.int8)
        lib().w4a8_gemm_w8_ref(_p(A), _p(W), C.c_int(M), C.c_int(N), C.c_int(K), _p(S))
    else:
        W = _c(W, np.uint8)
        lib().w4a8_gemm_w4_ref(_p(A), _p(W), C.c_int(M), C.c_int(N), C.c_int(K), _p(S))
    return S


def gemm_fast(A, W, w8, threads=1, pin=0, isa=-1, tile_lo=0, tile_hi=None, S=None):
    A = _c(A, np.int8)
    M, K = A.shape
    N = W.shape[0]
    W = np.ascontiguousarray(W).view(np.uint8)
    if S is None:
        S = np.zeros((M, N), np.int32)
    if tile_hi is None:
        tile_hi = N // 16
    used = lib().w4a8_gemm_fast(_p(A), _p(W), C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(int(w8)), _p(S),
                                C.c_int(tile_lo), C.c_int(tile_hi), C.c_int(threads), C.c_int(pin), C.c_int(isa))
    return S, used


def epilogue(S, a_scale, w_scale, w8):
    """S = sum a*w (int32 [M,N]) -> bf16 bits [M,N]."""
    S = _c(S, np.int32)
    M, N = S.shape
    a_scale = _c(a_scale, np.float32)
    w_scale = _c(w_scale, np.float32)
    out = np.empty((M, N), np.uint16)
    lib().w4a8_epilogue_all(_p(S), _p(a_scale), _p(w_scale), C.c_int(M), C.c_int(N), C.c_int(int(w8)), _p(out))
    return out


def linear(x_bits, W, ws, w8, threads=1, pin=0, want_c=True):
    """Whole dense linear: returns dict(q, as, S, C, isa)."""
    x = _c(x_bits, np.uint16)
    M, K = x.shape
    N = W.shape[0]
    W = np.ascontiguousarray(W).view(np.uint8)
    ws = _c(ws, np.float32)
    q = np.empty((M, K), np.int8)
    a_s = np.empty(M, np.float32)
    S = np.empty((M, N), np.int32)
    Cc = np.empty((M, N), np.uint16) if want_c else None
    isa = lib().w4a8_linear(_p(x), _p(W), _p(ws), C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(int(w8)), _p(q),
                            _p(a_s), _p(S), _p(Cc), C.c_int(threads), C.c_int(pin))
    return dict(q=q, a_scale=a_s, S=S, C=Cc, isa=isa)


def route(logits_bits, topk):
    lg = _c(logits_bits, np.uint16)
    T, E = lg.shape
    ids = np.empty((T, topk), np.int32)
    w = np.empty((T, topk), np.float32)
    rc = lib().w4a8_route(_p(lg), C.c_int(T), C.c_int(E), C.c_int(topk), _p(ids), _p(w))
    if rc != 0:
        raise ValueError("router width must be 16 * a power of two")
    return ids, w


def sort_layout(ids, E, tile_blocks):
    ids = _c(ids, np.int32)
    T, topk = ids.shape
    L = lib()
    rows_cap = L.w4a8_rows_cap(T, topk, E)
    tiles_cap = L.w4a8_tiles_cap(T, topk, E, tile_blocks)
    row_tok = np.full(rows_cap, -1, np.int32)
    route_pos = np.full(T * topk, -1, np.int32)
    te = np.zeros(tiles_cap, np.int32)
    t0 = np.zeros(tiles_cap, np.int32)
    tr = np.zeros(tiles_cap, np.int32)
    cnt = np.zeros(E, np.int32)
    meta = np.zeros(8, np.int32)
    L.w4a8_sort_layout(_p(ids), C.c_int(T), C.c_int(topk), C.c_int(E), C.c_int(tile_blocks), _p(row_tok), _p(route_pos),
                       _p(te), _p(t0), _p(tr), _p(cnt), _p(meta))
    nt, rows = int(meta[0]), int(meta[1])
    return dict(row_tok=row_tok[:rows].copy(), route_pos=route_pos.reshape(T, topk), tile_expert=te[:nt].copy(),
                tile_row0=t0[:nt].copy(), tile_rows=tr[:nt].copy(), expert_cnt=cnt, tiles=nt, rows=rows,
                rows_cap=rows_cap, tiles_cap=tiles_cap)


def silu_bf16_table():
    L = lib()
    return np.array([L.w4a8_silu_bf16(i) for i in range(65536)], dtype=np.uint16)


def silu_mul_quant(gu_bits):
    gu = _c(gu_bits, np.uint16)
    R, two_i = gu.shape
    I = two_i // 2
    q = np.empty((R, I), np.int8)
    s = np.empty(R, np.float32)
    p = np.empty((R, I), np.uint16)
    L = lib()
    for r in range(R):
        L.w4a8_silu_mul_quant_row(_p(gu[r]), C.c_int(I), _p(q[r]), _p(s[r:r + 1]), _p(p[r]))
    return q, s, p


def combine(Y_bits, topk_w, route_pos, H):
    Y = _c(Y_bits, np.uint16)
    w = _c(topk_w, np.float32)
    rp = _c(route_pos, np.int32)
    T, topk = w.shape
    out = np.empty((T, H), np.uint16)
    lib().w4a8_combine(_p(Y), _p(w), _p(rp), C.c_int(T), C.c_int(topk), C.c_int(H), _p(out))
    return out


def sigmoid(g):
    """The shared expert's gate: f32 sigmoid by the router's IEEE-only exp, elementwise."""
    g = np.ascontiguousarray(g, dtype=np.float32).ravel()
    L = lib()
    return np.array([L.w4a8_sigmoid(C.c_float(float(v))) for v in g], dtype=np.float32)


def combine_shared(Y_bits, topk_w, route_pos, sgate_bits, sh0, H):
    """combine() plus sigmoid(sgate[t]) * Y[sh0 + t]: the layer with a shared expert."""
    Y = _c(Y_bits, np.uint16)
    w = _c(topk_w, np.float32)
    rp = _c(route_pos, np.int32)
    sg = _c(sgate_bits, np.uint16)
    T, topk = w.shape
    out = np.empty((T, H), np.uint16)
    lib().w4a8_combine_shared(_p(Y), _p(w), _p(rp), _p(sg), C.c_int(int(sh0)), C.c_int(T), C.c_int(topk), C.c_int(H), _p(out))
    return out


def moe_layer(x_bits, topk_w, lay, Wgu, wsgu, Wdn, wsdn, I, threads=1, taps=False):
    """Whole expert layer. lay = sort_layout(...) dict. Returns dict(Y, out[, gu, q2, s2])."""
    x = _c(x_bits, np.uint16)
    T, H = x.shape
    E = lay["expert_cnt"].shape[0]
    topk = topk_w.shape[1]
    rows = lay["rows"]
    Y = np.zeros((rows, H), np.uint16)
    out = np.empty((T, H), np.uint16)
    gu = np.zeros((rows, 2 * I), np.uint16) if taps else None
    q2 = np.zeros((rows, I), np.int8) if taps else None
    s2 = np.zeros(rows, np.float32) if taps else None
    lib().w4a8_moe_layer(_p(x), C.c_int(T), C.c_int(H), C.c_int(I), C.c_int(E), C.c_int(topk),
                         _p(_c(topk_w, np.float32)), _p(_c(lay["route_pos"], np.int32)), _p(_c(lay["row_tok"], np.int32)),
                         _p(_c(lay["expert_cnt"], np.int32)), C.c_int(rows), _p(_c(Wgu, np.uint8)), _p(_c(wsgu, np.float32)),
                         _p(_c(Wdn, np.uint8)), _p(_c(wsdn, np.float32)), _p(Y), _p(out), _p(gu), _p(q2), _p(s2),
                         C.c_int(threads))
    return dict(Y=Y, out=out, gu=gu, q2=q2, s2=s2)


# ---------------------------------------------------------------------------- Hadamard-basis producers

def had32_rows(v, t):
    """f32 rows [M,K] (K % 32 == 0) -> rows transformed per 32-block."""
    v = np.array(v, dtype=np.float32, copy=True, order="C")
    M, K = v.shape
    lib().w4a8_had32_rows(_p(v), _p(_c(t, np.float32)), C.c_int(M), C.c_int(K))
    return v


def quant_had(x_bits, t):
    x = _c(x_bits, np.uint16)
    M, K = x.shape
    t = _c(t, np.float32)
    q, s = np.empty((M, K), np.int8), np.empty(M, np.float32)
    for m in range(M):
        lib().w4a8_quant_had_row(_p(x[m]), _p(t), C.c_int(K), _p(q[m]), _p(s[m:m + 1]))
    return q, s


def silu_mul_quant_had(gu_bits, t):
    gu = _c(gu_bits, np.uint16)
    M, I = gu.shape[0], gu.shape[1] // 2
    t = _c(t, np.float32)
    q, s = np.empty((M, I), np.int8), np.empty(M, np.float32)
    for m in range(M):
        lib().w4a8_silu_mul_quant_had_row(_p(gu[m]), _p(t), C.c_int(I), _p(q[m]), _p(s[m:m + 1]))
    return q, s


def add_rms_quant_had(y_bits, res_bits, w_bits, t, eps, threads_per_row=256):
    y, res, w = _c(y_bits, np.uint16), _c(res_bits, np.uint16), _c(w_bits, np.uint16)
    M, K = y.shape
    t = _c(t, np.float32)
    q, s, ro = np.empty((M, K), np.int8), np.empty(M, np.float32), np.empty((M, K), np.uint16)
    for m in range(M):
        lib().w4a8_add_rms_quant_had_row(_p(y[m]), _p(res[m]), _p(w), _p(t), C.c_int(K), C.c_float(eps),
                                         C.c_int(threads_per_row), _p(q[m]), _p(s[m:m + 1]), _p(ro[m]))
    return q, s, ro


def silu_f32_table():
    """f32 z / (1 + expf(-z)) of all 65,536 bf16 inputs, by the host's libm."""
    out = np.empty(65536, np.float32)
    lib().w4a8_silu_f32_table(_p(out))
    return out


def sigmoid_bf16_table():
    """bf16(1 / (1 + expf(-g))) of all 65,536 bf16 inputs."""
    f = lib().w4a8_sigmoid_bf16
    f.restype, f.argtypes = C.c_uint16, [C.c_uint16]
    return np.array([f(i) for i in range(65536)], dtype=np.uint16)


def gdn_norm_quant_had(x_bits, z_bits, w_bits, t, eps, silu_tab=None):
    """x [M,N] bf16 bits, z [M,N] (the rows the stride selects), w [128]; `silu_tab`: a card's own
    table of the f32 gate, or None for the host's libm."""
    x, z, w = _c(x_bits, np.uint16), _c(z_bits, np.uint16), _c(w_bits, np.uint16)
    M, N = x.shape
    t = _c(t, np.float32)
    tab = None if silu_tab is None else _c(silu_tab, np.float32)
    q, s = np.empty((M, N), np.int8), np.empty(M, np.float32)
    for m in range(M):
        lib().w4a8_gdn_norm_quant_had_row(_p(x[m]), _p(z[m]), _p(w), _p(t), _p(tab) if tab is not None else None,
                                          C.c_int(N), C.c_float(eps), _p(q[m]), _p(s[m:m + 1]))
    return q, s


def attn_gate_quant_had(core_bits, gate_bits, t, head_dim):
    """core [M,n]; gate [M, >= 2n]: the [q | gate] block rows."""
    core, gate = _c(core_bits, np.uint16), _c(gate_bits, np.uint16)
    M, n = core.shape
    t = _c(t, np.float32)
    q, s = np.empty((M, n), np.int8), np.empty(M, np.float32)
    for m in range(M):
        lib().w4a8_attn_gate_quant_had_row(_p(core[m]), _p(gate[m]), _p(t), C.c_int(n), C.c_int(head_dim),
                                           _p(q[m]), _p(s[m:m + 1]))
    return q, s
