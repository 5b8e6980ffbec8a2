"""Shared helpers of the parity tests."""
import numpy as np


def bits_equal(a, b):
    """Bit-for-bit equality of two fp32 arrays (distinguishes -0.0 from +0.0; NaNs equal when both NaN)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    if a.shape != b.shape:
        return False
    ai, bi = a.view(np.uint32), b.view(np.uint32)
    same = ai == bi
    both_nan = np.isnan(a) & np.isnan(b)
    return bool(np.all(same | both_nan))


def first_mismatch(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32).ravel()
    b = np.ascontiguousarray(b, dtype=np.float32).ravel()
    bad = np.nonzero((a.view(np.uint32) != b.view(np.uint32)) & ~(np.isnan(a) & np.isnan(b)))[0]
    if bad.size == 0:
        return "identical"
    i = int(bad[0])
    return "%d mismatches, first at %d: %r (0x%08x) vs %r (0x%08x)" % (
        bad.size, i, a[i], a.view(np.uint32)[i], b[i], b.view(np.uint32)[i])


def max_rel_err(y, ref):
    """max |y - ref| / max |ref|: the GEMM/conv acceptance metric (<= 1e-4)."""
    ref = np.asarray(ref, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    denom = np.abs(ref).max()
    return float(np.abs(y - ref).max() / (denom if denom > 0 else 1.0))


def to_np(t):
    return t.detach().cpu().numpy()


def unpack_bits(bits_words, K, N):
    """Packed 1-bit GEMM operand (uint32 words, [k_tiles][wide_groups][64 lanes][4]) -> int8 [K, N] of +-1.
    Word i of lane l: bit F + 8 c is column wide_group * 256 + F * 32 + l % 32, k = k_tile * 32 + (l / 32) * 16 + 4 i + c."""
    w = np.ascontiguousarray(bits_words).view(np.uint32)
    k_tiles = ((K + 255) // 256) * 8        # padded to a multiple of 8
    groups = (N + 255) // 256
    w = w.reshape(k_tiles, groups, 64, 4)
    out = np.ones((k_tiles * 32, groups * 256), np.int8)
    for lane in range(64):
        for i in range(4):
            for c in range(4):
                k_off = (lane >> 5) * 16 + 4 * i + c
                for F in range(8):
                    bit = (w[:, :, lane, i] >> np.uint32(F + 8 * c)) & np.uint32(1)   # [kt, group]
                    out[k_off::32, (F * 32 + (lane & 31))::256] = np.where(bit == 1, -1, 1)
    return out[:K, :N]


ONE_DIGIT_BIAS = 1024   # gemm_layout.hpp: a one-digit row stores its shift with this added


def unpack_digits(raw, M, K, with_one_digit=False):
    """Digit operand bytes -> (q int64 [M, K], shift int32 [M], row sums int64 [chunks, M]) as the kernels define it:
    fragments [row_block][k_tile][digit][lane][16 x int8], then the row sums ([chunks][rows] int64), then shifts.
    Shifts come back without the one-digit bias; with_one_digit appends the boolean mask of one-digit rows."""
    raw = np.ascontiguousarray(raw).view(np.uint8)
    rb, kt = (M + 31) // 32, ((K + 255) // 256) * 8
    rows, chunks = rb * 32, (K + 16383) // 16384
    nfrag = rb * kt * 3 * 1024
    d = raw[:nfrag].view(np.int8).reshape(rb, kt, 3, 64, 16).astype(np.int64)
    qf = d[:, :, 0] * 65536 + d[:, :, 1] * 256 + d[:, :, 2]          # [rb, kt, lane, j]
    q = np.zeros((rows, kt * 32), np.int64)
    for lane in range(64):
        for j in range(16):
            q[(lane & 31)::32, ((lane >> 5) * 16 + j)::32] = qf[:, :, lane, j]
    sums = raw[nfrag:nfrag + chunks * rows * 8].view(np.int64).reshape(chunks, rows)
    shift = raw[nfrag + chunks * rows * 8:nfrag + chunks * rows * 8 + rows * 4].view(np.int32)
    assert not q[M:].any() and not q[:, K:].any()
    shift = shift[:M].copy()
    one = shift >= ONE_DIGIT_BIAS // 2
    shift[one] -= ONE_DIGIT_BIAS
    if with_one_digit:
        lower = d[:, :, 1:].reshape(rb, kt, 2, 2, 32, 16).any(axis=(1, 2, 3, 5)).reshape(-1)[:M]   # per row
        assert not (lower & one).any(), "one-digit rows keep their value in the top digit"
        return q[:M, :K], shift, sums[:, :M].copy(), one
    return q[:M, :K], shift, sums[:, :M].copy()
