"""nz_encode_static (the entry point that allocates nothing) against nz_encode,
through the C ABI: container, packed stream, size and status must be
byte-identical, on two calls in a row that share the library's static scratch
(the second smaller, so it runs over what the first left behind)."""
import ctypes

import numpy as np
import pytest

from conftest import bf16_bits_normal, stress_bits

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _encode(bits, s, chunk, lane, static, norm_size=0):
    from neuzip_amd import _lib

    L = _lib.load()
    n = bits.size
    d_in = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = L.nz_exp_bound_bytes(n, chunk, lane)
    assert cap > 0
    comp = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    stored = L.nz_packed_stored_bytes(n, s, chunk, lane)
    packed = torch.zeros(max(8, stored), dtype=torch.uint8, device="cuda")
    aux = torch.zeros(4, dtype=torch.int64, device="cuda")
    norm = torch.zeros(L.nz_norm_bytes(n, norm_size) + 8, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    if static:
        rc = L.nz_encode_static(d_in.data_ptr(), n, s, chunk, lane, packed.data_ptr(), comp.data_ptr(), cap,
                                aux.data_ptr(), aux.data_ptr() + 8, norm_size, norm.data_ptr(), st)
    else:
        ws_bytes = L.nz_encode_workspace_bytes(n, chunk, lane)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        rc = L.nz_encode(d_in.data_ptr(), n, s, chunk, lane, packed.data_ptr(), comp.data_ptr(), cap,
                         ws.data_ptr(), ws_bytes, aux.data_ptr(), aux.data_ptr() + 8, None, norm_size,
                         norm.data_ptr(), st)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    total, status = int(aux[0].item()), int(aux[1].item()) & 0xFFFFFFFF
    return (comp[:total].cpu().numpy(), packed[:stored].cpu().numpy(), total, status,
            norm[: L.nz_norm_bytes(n, norm_size)].cpu().numpy())


@pytest.mark.parametrize("s,chunk,lane,norm_size", [(7, 131072, 256, 0), (3, 65536, 344, 64), (0, 32768, 64, 0)])
def test_static_scratch_encode_equals_nz_encode(oracle, s, chunk, lane, norm_size):
    from neuzip_amd import _lib

    L = _lib.load()
    first = stress_bits(300, 4099, seed=s)            # 1 229 700 elements, ragged
    second = bf16_bits_normal(70_001, seed=s + 1)     # smaller: reuses a corner of the same scratch
    if norm_size:
        first = np.where((first & 0x7F80) == 0x7F80, np.uint16(0x3F80), first).astype(np.uint16)
    for bits in (first, second):
        assert L.nz_encode_workspace_bytes(bits.size, chunk, lane) <= 16 << 20
        print(f"case static encode n={bits.size} s={s} chunk={chunk} lane={lane} norm={norm_size}", flush=True)
        got = _encode(bits, s, chunk, lane, True, norm_size)
        want = _encode(bits, s, chunk, lane, False, norm_size)
        assert got[2] == want[2] and got[3] == want[3] == 0
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
        assert np.array_equal(got[4], want[4])
        if not norm_size:  # and both are the oracle's bytes
            o_comp, o_packed = oracle.compress_bf16(bits, s, chunk, lane)
            assert np.array_equal(got[0], o_comp) and np.array_equal(got[1], o_packed)


def test_static_scratch_limit_is_reported():
    from neuzip_amd import _lib

    L = _lib.load()
    n = 8 << 20  # its encode scratch is beyond the static array
    assert L.nz_encode_workspace_bytes(n, 131072, 256) > 16 << 20
    d_in = torch.zeros(n, dtype=torch.int16, device="cuda")
    cap = L.nz_exp_bound_bytes(n, 131072, 256)
    comp = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    packed = torch.zeros(n, dtype=torch.uint8, device="cuda")
    aux = torch.zeros(4, dtype=torch.int64, device="cuda")
    rc = L.nz_encode_static(d_in.data_ptr(), n, 7, 131072, 256, packed.data_ptr(), comp.data_ptr(), cap,
                            aux.data_ptr(), aux.data_ptr() + 8, 0, None, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.ERR_CAPACITY and "NZ_STATIC_SCRATCH_BYTES" in _lib.last_error()
    torch.cuda.synchronize()
    assert int(aux[0].item()) == 0  # nothing ran
