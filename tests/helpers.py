"""Shared test utilities: seeded inputs, bit-pattern conversions, an independent
numpy statement of the quantiser and of the gfx950 layout."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)



class _LazyOracle:
    """The CPU oracle (the checker), imported on first use so that code which
    only wants the data generators does not load it."""

    def __getattr__(self, name):
        from oracle import wo_oracle

        return getattr(wo_oracle, name)


O = _LazyOracle()

F16, BF16 = 0, 1
DT_NAMES = {F16: "float16", BF16: "bfloat16"}


def torch_dtype(dt):
    import torch

    return torch.float16 if dt == F16 else torch.bfloat16


def bits_to_torch(bits_u16, dt, device="cpu"):
    """uint16 numpy bit patterns -> torch tensor of T."""
    import torch

    t = torch.from_numpy(np.ascontiguousarray(bits_u16).view(np.int16).copy())
    return t.view(torch_dtype(dt)).to(device)


def torch_to_bits(t):
    """torch tensor of T (any device) -> uint16 numpy bit patterns."""
    import torch

    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def f32_to_bits(a, dt):
    """float32 numpy -> T bit patterns, round-to-nearest-even, done by numpy
    (float16) or torch (bfloat16) rather than by the oracle."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if dt == F16:
        return a.astype(np.float16).view(np.uint16)
    import torch

    return torch.from_numpy(a).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()


def bits_to_f32(b, dt):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    if dt == F16:
        return b.view(np.float16).astype(np.float32)
    return (b.astype(np.uint32) << 16).view(np.float32)


def make_weight(K, N, dt, seed=1234, std=0.02, outlier_cols=0.0):
    """W ~ N(0, std) in fp32, optionally with a fraction of columns scaled x20,
    then cast to T (RNE): the weight_quantize input of the benchmark configurations."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((K, N), dtype=np.float32) * np.float32(std)
    if outlier_cols > 0:
        cols = rng.choice(N, size=int(np.ceil(outlier_cols * N)), replace=False)
        w[:, cols] *= np.float32(20.0)
    return f32_to_bits(w, dt)


def make_act(M, K, dt, seed=4321, dist="normal"):
    rng = np.random.default_rng(seed)
    if dist == "normal":
        x = rng.standard_normal((M, K), dtype=np.float32)
    else:
        x = rng.random((M, K), dtype=np.float32)
    return f32_to_bits(x, dt)


def make_bias(N, dt, seed=777, std=0.01):
    rng = np.random.default_rng(seed)
    return f32_to_bits(rng.standard_normal((N,), dtype=np.float32) * np.float32(std), dt)


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.sqrt((b * b).sum())
    return float(np.sqrt(((a - b) ** 2).sum()) / (den if den > 0 else 1.0))


# --------------------------------------------------------------------------
# Independent numpy statement of the quantiser (no code shared with the C
# oracle): abs-max / bound in fp32, cast with numpy/torch, fp32 divide, round
# half away from zero done in float64, clip.
# --------------------------------------------------------------------------
def np_quantize(w_bits, dt, bits, group_size):
    w = bits_to_f32(w_bits, dt)
    K, N = w.shape
    bound = np.float32(127.0 if bits == 8 else 7.0)
    g = K if group_size == -1 else group_size
    ng = (K + g - 1) // g
    scale_bits = np.empty((ng, N), np.uint16)
    q = np.empty((K, N), np.int32)
    with np.errstate(divide="ignore", invalid="ignore"):
        for gi in range(ng):
            blk = w[gi * g:(gi + 1) * g]
            amax = np.abs(blk).max(axis=0).astype(np.float32)
            if group_size == -1:
                # the per-channel maximum starts from the signed first element,
                # so an all-zero column keeps that element's sign of zero
                amax = np.where(amax == 0, blk[0], amax).astype(np.float32)
            s32 = (amax / bound).astype(np.float32)
            sb = f32_to_bits(s32, dt)
            scale_bits[gi] = sb
            s = bits_to_f32(sb, dt)
            r = (blk / s[None, :]).astype(np.float32).astype(np.float64)
            rounded = np.where(r >= 0, np.floor(r + 0.5), np.ceil(r - 0.5))
            if bits == 8:
                # NaN (0/0) -> 127 through the reference's min/max order
                c = np.where(np.isnan(rounded), 127.0, np.clip(rounded, -127.0, 127.0))
            else:
                # non-finite -> INT_MIN on x86 -> clipped to -7
                c = np.where(np.isfinite(rounded), np.clip(rounded, -7.0, 7.0), -7.0)
            q[gi * g:(gi + 1) * g] = c.astype(np.int32)
    if group_size == -1:
        scale_bits = scale_bits[0]
    return q, scale_bits


def np_quantize_llm_int8(w_bits, dt, group_size):
    """Independent statement of algo="llm.int8": np_quantize for int8 with the
    scale left as the fp32 quotient.  Returns (codes int32 [K,N], scale fp32)."""
    w = bits_to_f32(w_bits, dt)
    K, N = w.shape
    g = K if group_size == -1 else group_size
    ng = (K + g - 1) // g
    scale = np.empty((ng, N), np.float32)
    q = np.empty((K, N), np.int32)
    with np.errstate(divide="ignore", invalid="ignore"):
        for gi in range(ng):
            blk = w[gi * g:(gi + 1) * g]
            amax = np.abs(blk).max(axis=0).astype(np.float32)
            if group_size == -1:
                amax = np.where(amax == 0, blk[0], amax).astype(np.float32)
            s = (amax / np.float32(127.0)).astype(np.float32)
            scale[gi] = s
            r = (blk / s[None, :]).astype(np.float32).astype(np.float64)
            rounded = np.where(r >= 0, np.floor(r + 0.5), np.ceil(r - 0.5))
            c = np.where(np.isnan(rounded), 127.0, np.clip(rounded, -127.0, 127.0))
            q[gi * g:(gi + 1) * g] = c.astype(np.int32)
    return q, (scale[0] if group_size == -1 else scale)


def canonical_from_q(q, bits):
    """signed codes [K,N] -> canonical tensor ([K,N] int8 or [K,N/2] nibbles)."""
    if bits == 8:
        return q.astype(np.int8)
    lo = q[:, 0::2] & 0xF
    hi = q[:, 1::2] & 0xF
    return (lo | (hi << 4)).astype(np.uint8).view(np.int8)


def q_from_canonical(codes, bits):
    if bits == 8:
        return codes.astype(np.int32)
    b = codes.view(np.uint8).astype(np.int32)
    lo = b & 0xF
    hi = b >> 4
    lo = np.where(lo >= 8, lo - 16, lo)
    hi = np.where(hi >= 8, hi - 16, hi)
    K, H = codes.shape
    q = np.empty((K, H * 2), np.int32)
    q[:, 0::2] = lo
    q[:, 1::2] = hi
    return q


def paddle_hip_from_q(q, bits):
    """signed codes -> what a PADDLE_WITH_HIP build stores: transposed bytes,
    int4 nibbles +8."""
    if bits == 8:
        return np.ascontiguousarray(q.astype(np.int8).T)
    lo = (q[:, 0::2] + 8) & 0xF
    hi = (q[:, 1::2] + 8) & 0xF
    return np.ascontiguousarray((lo | (hi << 4)).astype(np.uint8).T).view(np.int8)


def gfx950_from_q(q, bits):
    """signed codes [K,N] -> the gfx950 streaming layout as a flat uint8 array.

    Strips of 16 columns; inside a strip, tiles of 64 k (int8) or 128 k (int4)
    of 1 KiB in which lane = 16*kb + j owns 16 bytes: column j, k values
    8*kb..8*kb+7 of each 32-deep k step.  int8 bytes are code+128 in k order;
    int4 packs a k step into one dword whose nibble p holds i = 2p (p < 4) or
    2(p-4)+1, as code+8.  K = 64 mod 128 ends with a 512-byte half tile."""
    K, N = q.shape
    T = N // 16
    if bits == 8:
        u = ((q + 128) & 0xFF).astype(np.uint8)
        # [kt, step, kb, i, tn, j] -> [tn, kt, kb, j, step, i]
        a = u.reshape(K // 64, 2, 4, 8, T, 16).transpose(4, 0, 2, 5, 1, 3)
        return np.ascontiguousarray(a).reshape(-1)
    u = ((q + 8) & 0xF).astype(np.uint32)
    pos = np.array([(i >> 1) + 4 * (i & 1) for i in range(8)], dtype=np.uint32)

    def pack_steps(block, nstep):
        # block: [nstep*32, N] -> dwords [tn, kb, j, step]
        b = block.reshape(nstep, 4, 8, T, 16)  # step, kb, i, tn, j
        dw = np.zeros((nstep, 4, T, 16), np.uint32)
        for i in range(8):
            dw |= b[:, :, i] << (4 * pos[i])
        return dw.transpose(2, 1, 3, 0)  # tn, kb, j, step

    full = K // 128
    parts = []
    if full:
        body = u[: full * 128].reshape(full, 128, N)
        tiles = np.stack([pack_steps(body[t], 4) for t in range(full)], axis=1)  # tn, kt, kb, j, step
        parts.append(np.ascontiguousarray(tiles).reshape(T, -1))
    if K % 128:
        tail = pack_steps(u[full * 128:], 2)  # tn, kb, j, step(2)
        parts.append(np.ascontiguousarray(tail).reshape(T, -1))
    strips = np.concatenate(parts, axis=1).astype("<u4")
    return np.ascontiguousarray(strips).view(np.uint8).reshape(-1)


def adversarial_weight(K, N, dt, seed=99):
    """A weight that exercises the quantiser's corner cases: an all-zero
    column, one starting with -0, exact .5 ties, values far below the fp16
    normal-scale range (subnormal scales), large magnitudes, one huge outlier,
    groups that are all zero."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((K, N)).astype(np.float32) * np.float32(0.02)
    w[:, 0] = 0.0
    w[:, 1] = 0.0
    w[0, 1] = -0.0
    w[:, 2] = 1e-4 * rng.standard_normal(K)  # fp16: scale < 2^-14, subnormal
    w[:, 3] = 3e-7 * rng.standard_normal(K)  # fp16: scale underflows towards 0
    w[:, 4] = 1000.0 * rng.standard_normal(K)
    w[:, 5] = np.where(np.arange(K) % 2 == 0, 0.5, 127.0)  # ties: 0.5 / 1.0 -> round up
    w[:, 6] = np.where(np.arange(K) % 3 == 0, -2.5, 127.0)
    w[:, 7] = 1e-3
    w[K // 2, 7] = 30000.0  # one outlier squeezes everything else to 0
    w[: min(K, 128), 8] = 0.0  # first group(s) all zero, rest not
    w[:, 9] = -np.abs(w[:, 9])  # negative first element
    w[:, 10] = np.linspace(-7, 7, K)
    w[:, 11] = np.linspace(-127, 127, K)
    w[:, 12] = 65504.0 * np.sign(rng.standard_normal(K))
    return f32_to_bits(w, dt)
