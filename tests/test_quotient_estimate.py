"""The rANS encoder on the GPU divides the state by a frequency with a float
multiplication (neuzip_amd/csrc/nz_kernels.hip, nz_rans_encode_body): q' =
trunc(float(x) * r) with r four units in the last place under the correctly
rounded 1 / f, then q = q' + (x - q' f >= f).  This pins the claim behind it in
IEEE float32 arithmetic on the host: for every frequency and states at and
around every kind of boundary, q' is the exact quotient or one less."""
import numpy as np


def _estimate(x, f):
    r = (np.float32(1.0) / f.astype(np.float32)).view(np.uint32) - np.uint32(4)
    p = x.astype(np.float32) * r.view(np.float32)  # uint32 -> float32 rounds to nearest even, like v_cvt_f32_u32
    return p.astype(np.uint32)                      # truncation, like v_cvt_u32_f32 on a non-negative value


def test_estimate_is_the_quotient_or_one_less():
    rng = np.random.default_rng(0)
    f = np.arange(1, 4097, dtype=np.uint64)[:, None]
    # quotients below 2^20 (the state is below f << 20 when it is divided): the extremes,
    # powers of two and their neighbours, and random ones
    q = np.unique(np.concatenate([
        np.array([0, 1, 2, 3, (1 << 20) - 1, (1 << 20) - 2], dtype=np.uint64),
        (1 << np.arange(1, 20, dtype=np.uint64)), (1 << np.arange(1, 20, dtype=np.uint64)) - 1,
        (1 << np.arange(1, 20, dtype=np.uint64)) + 1,
        rng.integers(0, 1 << 20, 1500, dtype=np.uint64)]))[None, :]
    for rem_kind in ("zero", "last", "random"):
        if rem_kind == "zero":
            rem = np.zeros_like(f)
        elif rem_kind == "last":
            rem = f - 1
        else:
            rem = rng.integers(0, 1 << 30, f.shape, dtype=np.uint64) % f
        x = q * f + rem
        assert int(x.max()) < 1 << 32
        est = _estimate(x.astype(np.uint32), np.broadcast_to(f, x.shape).astype(np.uint32)).astype(np.uint64)
        assert np.all(est <= q), rem_kind
        assert np.all(est + 1 >= q), rem_kind
        # the correction the kernel applies gives the exact quotient
        fixed = est + ((x - est * f) >= f)
        assert np.array_equal(fixed, np.broadcast_to(q, x.shape)), rem_kind
