"""Seeded synthetic tensors in raw GGUF block layouts for the MoE decode workloads.

Every generator returns numpy arrays of raw bytes exactly as they would sit in a
GGUF file (rows packed back to back, no padding), so the same bytes can be handed
to the device library and to a CPU checker.

Workload naming:
  C0  hidden 2048, 64 experts, top-8, ffn 512, gate/up/down Q8_0
  C2  hidden 2048, 512 experts, top-10, ffn 512, gate/up IQ3_S, down Q8_0,
      plus a Q8_0 shared expert gated by sigmoid(w.x)
"""
import numpy as np

F32, Q4_0, Q8_0, IQ4_NL, IQ3_S, IQ2_S = 0, 2, 8, 20, 21, 22

BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, IQ4_NL: 32, IQ3_S: 256, IQ2_S: 256, 14: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, IQ4_NL: 18, IQ3_S: 110, IQ2_S: 82, 14: 210}

BASE_SEED = 20261014


def row_bytes(t, cols):
    assert cols % BLOCK_ELEMS[t] == 0
    return cols // BLOCK_ELEMS[t] * BLOCK_BYTES[t]


def rng_for(seed, *stream):
    return np.random.Generator(np.random.Philox(key=seed, counter=[abs(hash_ints(stream)), 0, 0, 0]))


def hash_ints(vals):
    h = 1469598103934665603
    for v in vals:
        h = ((h ^ (int(v) & 0xFFFFFFFF)) * 1099511628211) & 0x7FFFFFFFFFFFFFFF
    return h


def _put_scales(blocks, scale_f32):
    """blocks: uint8 [..., block_bytes]; writes fp16(scale) into bytes 0..1."""
    h = scale_f32.astype(np.float16).view(np.uint16)
    blocks[..., 0] = (h & 0xFF).astype(np.uint8)
    blocks[..., 1] = (h >> 8).astype(np.uint8)


def q8_0_matrix(rng, rows, cols, sigma=0.02):
    nb = cols // 32
    blk = np.empty((rows, nb, 34), np.uint8)
    blk[..., 2:] = rng.integers(-127, 128, size=(rows, nb, 32), dtype=np.int8).view(np.uint8)
    _put_scales(blk, np.abs(rng.normal(0.0, sigma, size=(rows, nb))).astype(np.float32) / np.float32(127.0))
    return blk.reshape(rows, nb * 34)


def q4_0_matrix(rng, rows, cols, sigma=0.02):
    nb = cols // 32
    blk = np.empty((rows, nb, 18), np.uint8)
    blk[..., 2:] = rng.integers(0, 256, size=(rows, nb, 16), dtype=np.uint8)
    _put_scales(blk, np.abs(rng.normal(0.0, sigma, size=(rows, nb))).astype(np.float32) / np.float32(8.0))
    return blk.reshape(rows, nb * 18)


def iq4_nl_matrix(rng, rows, cols, sigma=0.02):
    nb = cols // 32
    blk = np.empty((rows, nb, 18), np.uint8)
    blk[..., 2:] = rng.integers(0, 256, size=(rows, nb, 16), dtype=np.uint8)
    _put_scales(blk, np.abs(rng.normal(0.0, sigma, size=(rows, nb))).astype(np.float32) / np.float32(127.0))
    return blk.reshape(rows, nb * 18)


def iq3_s_matrix(rng, rows, cols, sigma=0.01):
    nb = cols // 256
    blk = rng.integers(0, 256, size=(rows, nb, 110), dtype=np.uint8)
    _put_scales(blk, np.abs(rng.normal(0.0, sigma, size=(rows, nb))).astype(np.float32))
    return blk.reshape(rows, nb * 110)


def iq2_s_matrix(rng, rows, cols, sigma=0.01):
    nb = cols // 256
    blk = rng.integers(0, 256, size=(rows, nb, 82), dtype=np.uint8)
    _put_scales(blk, np.abs(rng.normal(0.0, sigma, size=(rows, nb))).astype(np.float32))
    return blk.reshape(rows, nb * 82)


Q6_K = 14


def q6_k_matrix(rng, rows, cols, sigma=0.02):
    """Q6_K super-blocks (210 bytes per 256 values: ql[128] qh[64] scales[16] d): uniform 6-bit codes, int8 sub-block scales
    uniform in [-64, 63], fp16 d = |N(0, sigma)| / 2048 at the end of the block."""
    nb = cols // 256
    blk = rng.integers(0, 256, size=(rows, nb, 210), dtype=np.uint8)
    blk[:, :, 192:208] = rng.integers(-64, 64, size=(rows, nb, 16), dtype=np.int8).view(np.uint8)
    d = (np.abs(rng.normal(0.0, sigma, size=(rows, nb))) / 2048.0).astype(np.float16)
    blk[:, :, 208:210] = d.view(np.uint8).reshape(rows, nb, 2)
    return blk.reshape(rows, nb * 210)


MATRIX_GEN = {Q8_0: q8_0_matrix, Q4_0: q4_0_matrix, IQ4_NL: iq4_nl_matrix, IQ3_S: iq3_s_matrix,
              IQ2_S: iq2_s_matrix, Q6_K: q6_k_matrix}


def matrix(t, rng, rows, cols):
    return MATRIX_GEN[t](rng, rows, cols)


def rms_normed(rng, n):
    x = rng.normal(0.0, 1.0, size=n).astype(np.float32)
    rms = np.sqrt(np.mean(x.astype(np.float64) ** 2))
    return (x / np.float32(rms)).astype(np.float32)


def make_layer(hidden, ffn, n_experts, top_k, gate_type, down_type, shared, seed=BASE_SEED, layer=0,
               router_sigma=None, up_type=None):
    """One MoE layer as a dict of numpy arrays (raw GGUF bytes for the quantised tensors)."""
    up_type = gate_type if up_type is None else up_type
    r = lambda tid: rng_for(seed, layer, tid)
    if router_sigma is None:
        router_sigma = 0.02
    L = dict(hidden=hidden, expert_ffn=ffn, n_experts=n_experts, top_k=top_k, w_scale=1.0,
             gate_type=gate_type, up_type=up_type, down_type=down_type)
    L["router"] = r(1).normal(0.0, router_sigma, size=(n_experts, hidden)).astype(np.float32)
    L["gate"] = matrix(gate_type, r(2), n_experts * ffn, hidden).reshape(n_experts, -1)
    L["up"] = matrix(up_type, r(3), n_experts * ffn, hidden).reshape(n_experts, -1)
    L["down"] = matrix(down_type, r(4), n_experts * hidden, ffn).reshape(n_experts, -1)
    if shared:
        L["shared_type"] = Q8_0
        L["shared_gate_inp"] = r(5).normal(0.0, 0.02, size=hidden).astype(np.float32)
        L["shared_gate"] = q8_0_matrix(r(6), ffn, hidden)
        L["shared_up"] = q8_0_matrix(r(7), ffn, hidden)
        L["shared_down"] = q8_0_matrix(r(8), hidden, ffn)
    else:
        L["shared_gate_inp"] = None
    return L


def make_c0(seed=BASE_SEED, layer=0):
    return make_layer(2048, 512, 64, 8, Q8_0, Q8_0, shared=False, seed=seed, layer=layer, router_sigma=0.02)


def make_c2(seed=BASE_SEED, layer=0, n_experts=512):
    # router rows ~ N(0, 1/sqrt(H)) so that logits of an RMS-normalised x are ~N(0,1)
    return make_layer(2048, 512, n_experts, 10, IQ3_S, Q8_0, shared=True, seed=seed, layer=layer,
                      router_sigma=1.0 / np.sqrt(2048.0))


def layer_bytes(L, k=None):
    """Algorithmic bytes one decode step of this layer must read."""
    H, F, E = L["hidden"], L["expert_ffn"], L["n_experts"]
    k = L["top_k"] if k is None else k
    per_expert = F * row_bytes(L["gate_type"], H) + F * row_bytes(L["up_type"], H) + H * row_bytes(L["down_type"], F)
    total = E * H * 4 + k * per_expert
    if L.get("shared_gate_inp") is not None:
        total += 2 * F * row_bytes(Q8_0, H) + H * row_bytes(Q8_0, F) + H * 4
    return total


def zipf_ids(rng, n_experts, k, s=1.1, perm=None):
    """k distinct expert ids drawn from Zipf(s) over a permutation of the experts."""
    p = 1.0 / np.arange(1, n_experts + 1, dtype=np.float64) ** s
    p /= p.sum()
    ranks = rng.choice(n_experts, size=k, replace=False, p=p)
    return (perm[ranks] if perm is not None else ranks).astype(np.int32)
