"""Random mixtures of manager calls against a shadow copy of what was written.

The manager holds small writes back and decodes weights ahead of their
requests; whatever the order of calls, a read has to return what the last
write under its handle held at the time of that write, bit for bit.
"""
import random

import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _weight(gen, rows, cols):
    return (torch.randn(rows, cols, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)


@pytest.mark.parametrize("seed", list(range(10)))
def test_random_calls_agree_with_a_shadow_copy(seed):
    import neuzip_amd

    rng = random.Random(seed)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    mgr = neuzip_amd.Manager(precision=7)
    if seed == 3:  # one run with every request and every write on its own
        mgr.decode_ahead = False
        mgr.write_behind = False
    shapes = [(64, 512), (128, 1024), (96, 512), (256, 1024), (33, 512), (512, 512), (200, 1024), (16, 512)]
    shadow, handles = {}, []
    for s in shapes:
        w = _weight(gen, *s)
        h = mgr.write(w)
        shadow[h] = w.clone()
        handles.append(h)
    side = torch.cuda.Stream()

    def check_read(h):
        got = mgr.read(h)
        assert got.shape == shadow[h].shape and torch.equal(got, shadow[h]), h

    for it in range(260):
        op = rng.random()
        h = rng.choice(handles)
        if op < 0.22:      # a pass over all handles in order, as a model would make it
            for hh in (handles if rng.random() < 0.7 else reversed(handles)):
                x = torch.randn(24, shadow[hh].shape[1], device="cuda", generator=gen).to(torch.bfloat16)
                with torch.no_grad():
                    assert torch.equal(mgr.linear(hh, x), torch.nn.functional.linear(x, shadow[hh])), (it, hh)
        elif op < 0.40:    # rewrite (same shape: in place), the source changed right afterwards
            w = _weight(gen, *shadow[h].shape)
            mgr.write(w, h)
            shadow[h] = w.clone()
            w.zero_()
        elif op < 0.46:    # rewrite with another shape
            w = _weight(gen, rng.choice([8, 40, 300]), rng.choice([512, 1024]))
            mgr.write(w, h)
            shadow[h] = w.clone()
        elif op < 0.52:    # several at once
            picks = rng.sample(handles, 3)
            ws = [_weight(gen, *shadow[p].shape) for p in picks]
            mgr.write_many(ws, picks)
            for p, w in zip(picks, ws):
                shadow[p] = w.clone()
        elif op < 0.70:
            check_read(h)
        elif op < 0.76:
            got = mgr.read_shared(h)
            assert torch.equal(got, shadow[h])
        elif op < 0.84:    # one activation row: the fused product (its own summation order)
            x = torch.randn(shadow[h].shape[1], device="cuda", generator=gen).to(torch.bfloat16)
            with torch.no_grad():
                got = mgr.linear(h, x).float()
            want = shadow[h].double() @ x.double()
            assert torch.allclose(got.double(), want, rtol=2e-2, atol=2e-3), (it, h)
        elif op < 0.88:
            assert mgr.size(h) > 0 and tuple(mgr.meta_dict[h]) == tuple(shadow[h].shape)
        elif op < 0.92:    # the update statement of the reference's training loop
            g = _weight(gen, *shadow[h].shape)
            mgr.write(mgr.read(h).add_(g, alpha=-0.5), h)
            shadow[h] = shadow[h].clone().add_(g, alpha=-0.5)
        elif op < 0.95:    # a call on another stream
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                w = _weight(gen, *shadow[h].shape)
                mgr.write(w, h)
                shadow[h] = w.clone()
                check_read(rng.choice(handles))
            torch.cuda.current_stream().wait_stream(side)
        elif op < 0.97:
            mgr.flush()
        else:
            mgr.trim()
    for h in handles:
        check_read(h)
    mgr._be.check()
