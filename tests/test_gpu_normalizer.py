"""Block normalizers on the GPU against the oracle (bit-exact: the float division
and product round like the oracle's)."""
import ctypes

import numpy as np
import pytest

from conftest import bf16_bits_normal, stress_bits
from test_gpu_parity import gpu_decode, gpu_encode

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _finite(bits):
    """NaN / Inf patterns replaced: the reference leaves their treatment open."""
    return np.where((bits & 0x7F80) == 0x7F80, np.uint16(0x3F80) | (bits & 0x8000), bits).astype(np.uint16)


def _dev(bits, shape=None):
    t = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16)
    return t.view(shape) if shape else t


def _bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)


@pytest.mark.parametrize("norm", [1, 2, 4, 8, 64, 512, 1024])
@pytest.mark.parametrize("s", [7, 3, 1, 0])
def test_encode_decode_match_oracle(oracle, norm, s):
    for n, kind in ((200_003, "stress"), (65536 * 2, "normal"), (5, "normal"), (1023, "stress")):
        bits = _finite(stress_bits(1, n, seed=n + s) if kind == "stress" else bf16_bits_normal(n, seed=norm))
        print(f"case norm={norm} s={s} n={n} {kind}", flush=True)
        comp, packed, nb = gpu_encode(bits, s, norm_size=norm)
        o_norm, o_scaled = oracle.block_normalize(bits, norm)
        assert np.array_equal(nb.cpu().numpy(), o_norm)
        o_comp, o_packed = oracle.compress_bf16(o_scaled, s, 131072, 256)
        assert np.array_equal(packed.cpu().numpy(), o_packed)
        assert np.array_equal(comp.cpu().numpy(), o_comp)
        rc, out = gpu_decode(comp, packed, n, s, norm_size=norm, norm=nb)
        assert rc == 0
        assert np.array_equal(out, oracle.reconstruct_normalized(bits, s, norm))


@pytest.mark.parametrize("e_big,e_x", [(1, 0), (1, 1), (2, 0), (8, 0), (9, 1), (127, 120), (254, 254), (254, 200)])
def test_every_mantissa_pair_on_the_gpu(oracle, e_big, e_x):
    """Groups of two [maximum with mantissa mb, element with mantissa mx] around the
    subnormal and overflow ranges: division, gradual underflow and rounding."""
    mb, mx = np.meshgrid(np.arange(128), np.arange(128), indexing="ij")
    big = ((e_big << 7) | mb).astype(np.uint16).reshape(-1)
    x = ((e_x << 7) | mx).astype(np.uint16).reshape(-1)
    x = np.where((x & 0x7FFF) > (big & 0x7FFF), big, x)
    x ^= np.uint16(0x8000) * (np.arange(x.size) % 2).astype(np.uint16)
    data = np.stack([big, x], axis=1).reshape(-1)
    comp, packed, nb = gpu_encode(data, 7, norm_size=2)
    o_norm, o_scaled = oracle.block_normalize(data, 2)
    assert np.array_equal(nb.cpu().numpy(), o_norm)
    rc, out = gpu_decode(comp, packed, data.size, 7, norm_size=2, norm=nb)
    assert rc == 0
    assert np.array_equal(out, oracle.block_denormalize(o_scaled, 2, o_norm))


@pytest.mark.parametrize("norm,precision", [(512, 3), (1024, 0), (8, 1), (64, 7)])
def test_manager_with_normalizers(oracle, tmp_path, norm, precision):
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=precision, normalizer_size=norm)
    shape = (300, 1024)
    bits = _finite(stress_bits(*shape, seed=norm))
    w = _dev(bits, shape)
    h = mgr.write(w)
    want = oracle.reconstruct_normalized(bits, precision, norm)
    assert np.array_equal(_bits(mgr.read(h)), want)
    o_norm, o_scaled = oracle.block_normalize(bits, norm)
    o_comp, o_packed = oracle.compress_bf16(o_scaled, precision, *mgr._be.geometry(h))
    assert mgr.size(h) == o_comp.size + o_packed.size + o_norm.size  # cuda/high_level.cu:208-221
    # split: exponent and sign|mantissa bytes of the normalized tensor, precision 7 (high_level.cu:289)
    e, f = mgr.split(w)
    oe, of = oracle.split(o_scaled, 7)
    assert np.array_equal(e.cpu().numpy().reshape(-1), oe) and np.array_equal(f.cpu().numpy().reshape(-1), of)
    # linear, batched read, fused product
    w_rec = _dev(want, shape)
    x = torch.randn(4, 1024, device="cuda").to(torch.bfloat16)
    assert torch.equal(mgr.linear(h, x), torch.nn.functional.linear(x, w_rec))
    h2 = mgr.write(_dev(_finite(bf16_bits_normal(70_000, 2))))
    outs = [torch.zeros(300 * 1024, dtype=torch.bfloat16, device="cuda"),
            torch.zeros(70_000, dtype=torch.bfloat16, device="cuda")]
    mgr._be.read_batch(mgr._be.batch_plan([h, h2]), outs)
    assert np.array_equal(_bits(outs[0]), want)
    assert torch.equal(outs[1], mgr.read(h2))
    y = torch.zeros(300, dtype=torch.bfloat16, device="cuda")
    names = (ctypes.c_char_p * 1)(h.encode())
    mgr._be.gemv_batch(names, x[0].contiguous(), None, [y])
    ref = w_rec.double() @ x[0].double()
    tol = 2.0 ** -8 * ref.abs() + 1e-5 * (w_rec.double().abs() @ x[0].double().abs())
    assert bool(((y.double() - ref).abs() <= tol).all())
    # checkpoint round trip keeps the group bytes
    mgr.save(tmp_path / "n.pt")
    other = neuzip_amd.Manager(precision=precision, normalizer_size=norm)
    other.load(tmp_path / "n.pt")
    assert np.array_equal(_bits(other.read(h)), want) and other.size(h) == mgr.size(h)
    with pytest.raises(RuntimeError, match="normalizer_size"):
        neuzip_amd.Manager(precision=precision).load(tmp_path / "n.pt")
    mgr._be.check()
    other._be.check()
