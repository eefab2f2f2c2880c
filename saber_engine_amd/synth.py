"""Seeded synthetic operands of the W4A8-iu8 linear, as the benchmark configurations
describe them: one PRNG stream per case, drawn in the order W -> ws -> A.

  W4  int4 codes uniform in [-8, 7], logical [N, K]; canonical storage row-major,
      two codes a byte along K, low nibble = even k (the export form the reference's
      graph records, crates/saber-model/src/graph.rs:2591-2592)
  W8  int8 uniform in [-127, 127], row-major [N, K]
  ws  f32 |N(0, 0.02)| + 1e-4, [N]
  A   bf16 N(0, 1) [M, K]; floor(0.005 K) channels (columns), chosen once per tensor,
      scaled x20 before the bf16 rounding
"""
import numpy as np


def f32_to_bf16_bits(x):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16); finite inputs."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_w4(codes):
    """int8 codes in [-8,7], [N,K] -> canonical nibbles uint8 [N,K/2]."""
    c = codes.astype(np.uint8) & 15
    return (c[:, 0::2] | (c[:, 1::2] << 4)).astype(np.uint8)


def unpack_w4(w4):
    """canonical nibbles uint8 [N,K/2] -> int8 codes [N,K]."""
    lo = (w4 & 15).astype(np.int8)
    hi = (w4 >> 4).astype(np.int8)
    lo = np.where(lo >= 8, lo - 16, lo).astype(np.int8)
    hi = np.where(hi >= 8, hi - 16, hi).astype(np.int8)
    out = np.empty((w4.shape[0], w4.shape[1] * 2), np.int8)
    out[:, 0::2] = lo
    out[:, 1::2] = hi
    return out


def weights(rng, N, K, w8):
    if w8:
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    else:
        W = pack_w4(rng.integers(-8, 8, size=(N, K), dtype=np.int8))
    ws = (np.abs(rng.normal(0.0, 0.02, size=N)) + 1e-4).astype(np.float32)
    return W, ws


def activations(rng, M, K):
    a = rng.standard_normal(size=(M, K), dtype=np.float32)
    n_out = int(0.005 * K)
    if n_out:
        cols = rng.choice(K, size=n_out, replace=False)
        a[:, cols] *= 20.0
    return f32_to_bf16_bits(a)


def dense_case(M, N, K, w8=False, seed=0):
    """Returns dict(W, ws, X) with X the bf16 bit patterns [M,K]."""
    rng = np.random.default_rng(seed)
    W, ws = weights(rng, N, K, w8)
    X = activations(rng, M, K)
    return dict(W=W, ws=ws, X=X, M=M, N=N, K=K, w8=bool(w8))


def moe_case(T, E=128, topk=8, H=4096, I=1536, seed=0, experts=None):
    """Expert layer operands: per-expert gate_up W4 [2I,H] and down W4 [H,I] with row
    scales, activations x bf16 [T,H], router logits bf16 N(0,1) [T,E].
    `experts` limits how many experts get distinct weights (the rest alias them
    round-robin) so that small tests do not draw E full matrices."""
    rng = np.random.default_rng(seed)
    ne = E if experts is None else min(E, experts)
    Wgu = np.empty((ne, 2 * I, H // 2), np.uint8)
    wsgu = np.empty((ne, 2 * I), np.float32)
    Wdn = np.empty((ne, H, I // 2), np.uint8)
    wsdn = np.empty((ne, H), np.float32)
    for e in range(ne):
        Wgu[e], wsgu[e] = weights(rng, 2 * I, H, False)
        Wdn[e], wsdn[e] = weights(rng, H, I, False)
    if ne < E:
        idx = np.arange(E) % ne
        Wgu, wsgu, Wdn, wsdn = Wgu[idx], wsgu[idx], Wdn[idx], wsdn[idx]
    X = activations(rng, T, H)
    logits = f32_to_bf16_bits(rng.standard_normal(size=(T, E), dtype=np.float32))
    return dict(Wgu=Wgu, wsgu=wsgu, Wdn=Wdn, wsdn=wsdn, X=X, logits=logits, T=T, E=E, topk=topk, H=H, I=I)


# The decoder-layer linears of the benchmark configurations (TP=1, hidden 5120).
LAYER_LINEARS = (
    ("qkv", 7168, 5120),
    ("o", 5120, 5120),
    ("gate_up", 34816, 5120),
    ("down", 5120, 17408),
)

# The 64-entry mixed launch sequence: 19 int8-row linears among 64, on output-side
# projections (N = 5120), mirroring the reference's promoted set as a fraction
# (crates/saber-exec/tests/macaq_iu8.rs:48-65).
def mixed_sequence():
    seq = []
    names = [l for l in LAYER_LINEARS]
    w8_slots = {1, 3, 5, 7, 9, 11, 13, 17, 21, 25, 29, 33, 37, 41, 45, 49, 53, 57, 61}
    for i in range(64):
        name, n, k = names[i % 4]
        w8 = i in w8_slots and name in ("o", "down")
        seq.append((name, n, k, w8))
    # every W8 slot must be an output-side projection: slots above are odd -> "o"/"down"
    assert sum(1 for s in seq if s[3]) == 19
    return seq
