"""Seeded synthetic operands for the W4A16 linear op (harness side; no device code).

The generator is SplitMix64 with the constants of the reference's parity gate
(crates/server/src/probes/w4a16/gates.rs:182-196).  Because SplitMix64's state is an arithmetic sequence
(state_i = seed + i * GAMMA), the i-th output is computed directly, which lets numpy produce the hundreds of millions
of nibbles the layer shapes need.  `SplitMix64.next()` and the vectorised `stream()` return the same sequence.

Operand formats (crates/core/src/quant/lane.rs:62-63, scripts/gen_tiny_w4a16.py:44-48):
  q  u32 [n][k/8]   element i of a row is nibble (q[i>>3] >> 4*(i&7)) & 0xF, weight value = nibble - 8
  s  u16 [n][k/g]   one f16 (or bf16) scale per group of g elements along k
  x  u16 [t][k]     f16 activations
"""
import numpy as np

GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
GATE_SEED = 0x9E3779B97F4A7C15  # default seed of the reference gate (gates.rs:13)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


class SplitMix64:
    """Scalar generator, same stepping as gates.rs:187-193."""

    def __init__(self, seed):
        self.state = int(seed) & 0xFFFFFFFFFFFFFFFF
        self.count = 0

    def next(self):
        self.state = (self.state + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & 0xFFFFFFFFFFFFFFFF
        return z ^ (z >> 31)

    def next_pm1(self):
        """Uniform in [-1, 1) with 24 random bits, as gates.rs:194-196."""
        return np.float32(np.float32(self.next() >> 40) / np.float32(1 << 24)) * np.float32(2.0) - np.float32(1.0)


def stream(seed, count, offset=0):
    """Outputs offset .. offset+count-1 of SplitMix64(seed) as uint64."""
    with np.errstate(over="ignore"):
        i = np.arange(offset + 1, offset + count + 1, dtype=np.uint64)
        return _mix(np.uint64(int(seed) & 0xFFFFFFFFFFFFFFFF) + i * GAMMA)


def shape_seed(n, k, seed=GATE_SEED, tensor=0):
    """Per-shape seed as gates.rs:108, plus a tensor index so q / s / x draw from separate streams."""
    return (int(seed) ^ (int(n) << 32) ^ int(k) ^ (int(tensor) * 0xD1B54A32D192ED03)) & 0xFFFFFFFFFFFFFFFF


def f32_to_f16_bits(v):
    """f32 -> f16 bit patterns, round to nearest even (numpy's cast; equals the reference f32_to_f16,
    crates/backend-gpu/src/rawcuda/w4a16_dec/mod.rs:187-219, for every non-NaN input)."""
    return np.asarray(v, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(h):
    return np.asarray(h, dtype=np.uint16).view(np.float16).astype(np.float32)


def uniform01(seed, count):
    """Uniform [0,1) f32 with 24 random bits."""
    return (stream(seed, count) >> np.uint64(40)).astype(np.float32) / np.float32(1 << 24)


def gate_x(n, k, t, seed=GATE_SEED):
    """Activations of the reference parity gate: uniform (-1,1) rounded to f16 (gates.rs:108-111)."""
    u = uniform01(seed ^ (n << 32) ^ k, t * k)
    return f32_to_f16_bits(u * np.float32(2.0) - np.float32(1.0)).reshape(t, k)


def normal_f16(seed, shape):
    """N(0,1) by Box-Muller from two uniform streams, rounded to f16."""
    count = int(np.prod(shape))
    half = (count + 1) // 2
    r = stream(seed, 2 * half)
    u1 = ((r[:half] >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)  # (0,1]
    u2 = (r[half:] >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    rad = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([rad * np.cos(2.0 * np.pi * u2), rad * np.sin(2.0 * np.pi * u2)])[:count]
    return f32_to_f16_bits(z.astype(np.float32)).reshape(shape)


def normal_f32(seed, shape):
    count = int(np.prod(shape))
    half = (count + 1) // 2
    r = stream(seed, 2 * half)
    u1 = ((r[:half] >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)
    u2 = (r[half:] >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    rad = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([rad * np.cos(2.0 * np.pi * u2), rad * np.sin(2.0 * np.pi * u2)])[:count]
    return z.astype(np.float32).reshape(shape)


def weights_q(seed, n, k):
    """Packed int4 weights, u32 [n][k/8]: each word is the low 32 bits of one generator output, i.e. eight
    independent uniform nibbles (weight values uniform in -8..7)."""
    assert k % 8 == 0
    return (stream(seed, n * (k // 8)) & np.uint64(0xFFFFFFFF)).astype(np.uint32).reshape(n, k // 8)


def scales_f16(seed, n, k, group, lo=0.002, hi=0.02):
    """f16 scales uniform in [lo, hi), u16 [n][k/group]."""
    u = uniform01(seed, n * (k // group))
    return f32_to_f16_bits(np.float32(lo) + np.float32(hi - lo) * u).reshape(n, k // group)


def pack_nibbles(vals):
    """int array [n][k] of values in -8..7 -> u32 [n][k/8] in the reference pack order
    (element i at bits 4*(i&7) of word i>>3, offset-binary nibble = value + 8)."""
    v = (np.asarray(vals).astype(np.int64) + 8).astype(np.uint32)
    assert v.min() >= 0 and v.max() <= 15
    n, k = v.shape
    v = v.reshape(n, k // 8, 8)
    sh = (np.arange(8, dtype=np.uint32) * 4)[None, None, :]
    return np.bitwise_or.reduce(v << sh, axis=2).astype(np.uint32)


def unpack_nibbles(q, k):
    """u32 [n][k/8] -> int8 [n][k] weight values (nibble - 8)."""
    q = np.asarray(q, dtype=np.uint32)
    sh = (np.arange(8, dtype=np.uint32) * 4)[None, None, :]
    nib = (q[:, :, None] >> sh) & np.uint32(0xF)
    return (nib.astype(np.int8) - 8).reshape(q.shape[0], k)


def make_linear(n, k, group, t, seed=GATE_SEED, x_dist="normal"):
    """One synthetic linear: (q u32[n][k/8], s u16[n][k/g], x u16[t][k])."""
    q = weights_q(shape_seed(n, k, seed, 1), n, k)
    s = scales_f16(shape_seed(n, k, seed, 2), n, k, group)
    if x_dist == "normal":
        x = normal_f16(shape_seed(n, k, seed, 3), (t, k))
    else:
        x = gate_x(n, k, t, seed)
    return q, s, x


def make_experts(n_exp, h, n_ff, group, seed=GATE_SEED):
    """Synthetic experts of one MoE layer: q13 u32 [E][2*n_ff][h/8] (gate rows then up rows), s13 u16 [E][2*n_ff][h/g],
    q2 u32 [E][h][n_ff/8], s2 u16 [E][h][n_ff/g]; distributions as for a dense linear."""
    q13 = weights_q(shape_seed(2 * n_ff, h, seed, 11), n_exp * 2 * n_ff, h).reshape(n_exp, 2 * n_ff, h // 8)
    s13 = scales_f16(shape_seed(2 * n_ff, h, seed, 12), n_exp * 2 * n_ff, h, group).reshape(n_exp, 2 * n_ff, h // group)
    q2 = weights_q(shape_seed(h, n_ff, seed, 13), n_exp * h, n_ff).reshape(n_exp, h, n_ff // 8)
    s2 = scales_f16(shape_seed(h, n_ff, seed, 14), n_exp * h, n_ff, group).reshape(n_exp, h, n_ff // group)
    return q13, s13, q2, s2


def router_logits(t, n_exp, seed=GATE_SEED):
    """Router logits f32 [t][n_exp], N(0,1)."""
    return normal_f32(shape_seed(n_exp, t, seed, 15), (t, n_exp))
