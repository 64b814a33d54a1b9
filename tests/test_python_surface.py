"""CPU: the Python surface (module conversion, Parameter, CompressedLinear,
update hooks) against torch reference semantics, with a dense stand-in for the
native manager so that no GPU is needed.  Mirrors neuzip/utils.py:57-68,
neuzip/nn/*.py, neuzip/ops/linear.py and neuzip/__init__.py:16-35."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import neuzip_amd
from neuzip_amd.nn import Linear, Parameter
from neuzip_amd.utils import _convert


class FakeManager:
    """CPU manager with the oracle's reconstruction as storage semantics."""

    def __init__(self, oracle, precision=7):
        self.o, self.s = oracle, precision
        self.meta_dict, self.store, self.writes = {}, {}, []

    def write(self, tensor, handle=None):
        key = str(len(self.meta_dict)) if handle is None else handle
        self.meta_dict[key] = tensor.shape
        bits = tensor.detach().contiguous().view(torch.int16).numpy().view(np.uint16).reshape(-1)
        rec = self.o.reconstruct(bits, self.s)
        self.store[key] = torch.from_numpy(rec.view(np.int16).copy()).view(torch.bfloat16)
        self.writes.append(key)
        return key

    def read(self, handle):
        return self.store[handle].clone().reshape(self.meta_dict[handle])

    def size(self, handle):
        return self.store[handle].numel()

    def linear(self, handle, inputs, bias=None):
        return torch.nn.functional.linear(inputs, self.read(handle), bias)

    def convert(self, module):
        return _convert(self, module)


class Block(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.attn = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.ReLU(), torch.nn.Linear(8, 8, bias=False))
        self.norm = torch.nn.LayerNorm(8)


class Toy(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = torch.nn.Embedding(11, 8)
        self.layers = torch.nn.ModuleList([Block(), Block()])
        self.lm_head = torch.nn.Linear(8, 11, bias=False)
        self.my_lm_head_proj = torch.nn.Linear(8, 8)


def test_convert_structure(oracle):
    model = Toy().to(torch.bfloat16)
    mgr = FakeManager(oracle)
    out = mgr.convert(model)
    assert out is model
    # every nn.Linear outside names containing "lm_head" is swapped; embeddings are not
    assert isinstance(model.lm_head, torch.nn.Linear)
    assert isinstance(model.my_lm_head_proj, torch.nn.Linear)
    assert isinstance(model.embed, torch.nn.Embedding)
    converted = [m for m in model.modules() if isinstance(m, Linear)]
    assert len(converted) == 4
    assert sorted(mgr.meta_dict) == ["0", "1", "2", "3"]  # handles are str(len(meta_dict))
    for m in converted:
        assert isinstance(m.weight, Parameter) and m.weight is m._p
        assert m.weight.numel() == 0 and m.weight.dtype == torch.bfloat16
        assert m.weight._shape == (m.out_features, m.in_features)
        assert repr(m).startswith("Linear(! in_features=")
    assert model.layers[0].attn[2].bias is None and model.layers[0].attn[0].bias is not None


def test_conv1d_is_recognised(oracle):
    Conv1D = pytest.importorskip("transformers.pytorch_utils").Conv1D
    from neuzip_amd.utils import _convertible_types

    assert Conv1D in _convertible_types() and torch.nn.Linear in _convertible_types()


@pytest.mark.parametrize("precision", (7, 3))
def test_forward_backward_match_dense_linear(oracle, precision):
    torch.manual_seed(0)
    dense = torch.nn.Linear(16, 12).to(torch.bfloat16)
    dense.weight.data.normal_(0, 0.02)
    mgr = FakeManager(oracle, precision)
    comp = Linear(mgr, dense)
    w_rec = mgr.read("0")
    ref = torch.nn.Linear(16, 12).to(torch.bfloat16)
    ref.weight.data.copy_(w_rec)
    ref.bias.data.copy_(dense.bias.data)

    x = torch.randn(3, 5, 16, dtype=torch.bfloat16)
    x1, x2 = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    y1, y2 = comp(x1), ref(x2)
    assert torch.equal(y1, y2)
    g = torch.randn_like(y1)
    y1.backward(g)
    y2.backward(g)
    assert torch.equal(x1.grad, x2.grad)
    assert torch.equal(comp.bias.grad, ref.bias.grad)
    # weight gradient accumulates on _gradient, autograd only sees a zero-size dummy
    assert torch.equal(comp.weight._gradient, ref.weight.grad)
    assert comp.weight.grad is not None and comp.weight.grad.numel() == 0
    y1b = comp(x1)
    y1b.backward(g)
    assert torch.equal(comp.weight._gradient, 2 * ref.weight.grad)


def test_autocast_cast_and_grad_dtype(oracle):
    dense = torch.nn.Linear(8, 4, bias=False).to(torch.bfloat16)
    comp = Linear(FakeManager(oracle), dense)
    x = torch.randn(2, 8, dtype=torch.float32, requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=True):
        if not torch.is_autocast_enabled():
            pytest.skip("autocast flag cannot be enabled without a GPU build")
        y = comp(x)
    assert y.dtype == torch.bfloat16
    y.float().sum().backward()
    assert x.grad.dtype == torch.float32  # cast back to the caller's dtype (ops/linear.py:34)


class _Sched:
    def __init__(self, lr):
        self.lr = lr

    def get_last_lr(self):
        return [self.lr]


def test_compressed_lomo_hook(oracle):
    torch.manual_seed(1)
    dense = torch.nn.Linear(8, 8, bias=False).to(torch.bfloat16)
    mgr = FakeManager(oracle, 7)
    comp = Linear(mgr, dense)
    p = comp.weight
    w0 = mgr.read(p._handle)
    neuzip_amd.compressed_lomo_hook(_Sched(0.5), p)  # no gradient yet: nothing happens
    assert mgr.writes == ["0"]
    p._gradient = torch.ones(8, 8, dtype=torch.bfloat16)
    neuzip_amd.compressed_lomo_hook(_Sched(0.5), p)
    assert mgr.writes == ["0", "0"]  # rewritten under the same handle
    assert p._gradient is None and p.grad is None
    assert torch.equal(mgr.read(p._handle), w0 - 0.5)


def test_post_accumulate_hook_fires(oracle):
    torch.manual_seed(2)
    dense = torch.nn.Linear(8, 8).to(torch.bfloat16)
    mgr = FakeManager(oracle, 7)
    comp = Linear(mgr, dense)
    w0 = mgr.read("0")
    from functools import partial

    comp.weight.register_post_accumulate_grad_hook(partial(neuzip_amd.compressed_lomo_hook, _Sched(0.25)))
    x = torch.randn(4, 8, dtype=torch.bfloat16)
    comp(x).float().sum().backward()
    gw = torch.mm(torch.ones(4, 8, dtype=torch.bfloat16).t(), x)
    assert torch.equal(mgr.read("0"), w0 - 0.25 * gw)
    assert comp.weight._gradient is None


def test_lomo_hook_dense():
    p = torch.nn.Parameter(torch.ones(3))
    neuzip_amd.lomo_hook(_Sched(0.1), p)  # no grad: no-op
    p.grad = torch.full((3,), 2.0)
    neuzip_amd.lomo_hook(_Sched(0.1), p)
    assert torch.allclose(p.data, torch.full((3,), 0.8)) and p.grad is None


def test_manager_argument_errors():
    A = neuzip_amd.Algorithm
    assert {m.name for m in A} == {"ans", "gdeflate", "zstd", "dummy"}  # neuzip/binding.py:23-27
    with pytest.raises(AttributeError, match="Manager_f5_n0"):
        neuzip_amd.Manager(precision=5)
    with pytest.raises(AttributeError, match="Manager_f7_n3"):
        neuzip_amd.Manager(normalizer_size=3)
    with pytest.raises(RuntimeError, match="Unsupported algorithm"):
        neuzip_amd.Manager(algorithm=A.zstd)


def test_reference_package_name_is_importable():
    """``import neuzip`` exposes the reference's surface (neuzip/__init__.py:8-13)
    and module paths, and its Manager keeps the reference's constructor
    signature (neuzip/binding.py:56-62)."""
    import inspect

    import neuzip
    import neuzip.binding
    import neuzip.nn.embedding
    import neuzip.nn.linear
    import neuzip.nn.module
    import neuzip.ops.linear
    import neuzip.utils

    assert neuzip.__all__ == ["ops", "nn", "Algorithm", "Manager"]
    for name in neuzip.__all__ + ["lomo_hook", "compressed_lomo_hook"]:
        assert hasattr(neuzip, name)
    assert neuzip.nn is neuzip_amd.nn and neuzip.ops is neuzip_amd.ops
    assert neuzip.nn.Linear is Linear and neuzip.nn.Parameter is Parameter
    assert neuzip.nn.linear.Linear is Linear and neuzip.nn.module.Parameter is Parameter
    assert neuzip.ops.CompressedLinear is neuzip_amd.ops.CompressedLinear
    assert neuzip.ops.linear.CompressedLinear is neuzip_amd.ops.CompressedLinear
    assert neuzip.utils._convert is _convert
    assert neuzip.binding.Manager is neuzip.Manager and issubclass(neuzip.Manager, neuzip_amd.Manager)
    assert [m.name for m in neuzip.Algorithm] == ["ans", "gdeflate", "zstd", "dummy"]  # neuzip/binding.py:23-27
    params = inspect.signature(neuzip.Manager.__init__).parameters
    assert list(params)[:5] == ["self", "algorithm", "precision", "normalizer_size", "chunk_size"]
    assert params["algorithm"].default is neuzip.Algorithm.ans and params["precision"].default == 7
    assert params["normalizer_size"].default is None and params["chunk_size"].default == 2 ** 16
    # the dense pass-through needs no device: convert() runs as the reference words it
    mgr = neuzip.Manager(algorithm=neuzip.Algorithm.dummy)
    assert mgr.meta_dict == {} and callable(mgr.convert)
    with pytest.raises(AttributeError, match="Manager_f5_n0"):
        neuzip.Manager(precision=5)


def test_group_geometry_choice_is_one_round_of_workgroups():
    """FusedGemv picks, for matrices that one launch decodes together, a geometry
    under which their chunks are at most three per compute unit in total and
    the estimated stored size stays inside the manager's budget, and stores
    them again only when that differs from what they have (host logic, no GPU:
    a stand-in backend records the calls)."""
    from neuzip_amd.fused import FusedGemv, _Group

    class Be:
        auto_geometry = True

        def __init__(self, sizes, geo, size_budget=1.01):
            self.sizes, self.geo, self.hints, self.size_budget = sizes, dict(geo), {}, size_budget

        def estimated_size_ratio(self, n, chunk, lane):
            full, rest = divmod(n, chunk)
            segs = full * -(-chunk // (64 * lane)) + -(-rest // (64 * lane))
            return 1.0008 + (134.4 * segs + 78.0 * (full + (rest > 0)) + 600.0) / n

        def in_budget(self, n, chunk, lane):
            return self.estimated_size_ratio(n, chunk, lane) + 0.0003 <= self.size_budget

        def numel(self, h):
            return self.sizes[h]

        def geometry(self, h):
            return self.geo[h]

        def geometry_hint(self, h, chunk, lane):
            self.hints[h] = (chunk, lane)

    class Mgr:
        def __init__(self, be):
            self._be, self.written = be, []

        def read(self, h):
            return h

        def write(self, dense, h):
            self.written.append(h)
            self._be.geo[h] = self._be.hints[h]

    def group_of(handles):
        g = _Group.__new__(_Group)
        g.handles = handles
        return g

    cus = 256
    for sizes, budget in (({"gate": 14336 * 4096, "up": 14336 * 4096}, 1.01),            # 8B-shaped gate / up
                          ({"q": 4096 * 4096, "k": 1024 * 4096, "v": 1024 * 4096}, 1.05),  # q / k / v
                          ({"a": 3_000_000, "b": 5_000_001}, 1.05)):
        be = Be(sizes, {h: (131072, 256) for h in sizes}, budget)
        f = FusedGemv.__new__(FusedGemv)
        f.manager = Mgr(be)
        f._fit_geometry(group_of(list(sizes)), cus=cus)
        geos = {be.geo[h] for h in sizes}
        assert len(geos) == 1
        chunk, lane = geos.pop()
        assert chunk == 512 * lane and 64 <= lane <= 512 and lane % 8 == 0
        assert all(be.in_budget(n, chunk, lane) for n in sizes.values())
        chunks = sum(-(-n // chunk) for n in sizes.values())
        assert chunks <= 3 * cus
        assert sorted(f.manager.written) == sorted(sizes)
        f._fit_geometry(group_of(list(sizes)), cus=cus)            # already fitted: nothing is stored again
        assert sorted(f.manager.written) == sorted(sizes)
    # gate / up of the 8B shape: 2 x 378 chunks of 304 symbols per lane
    be = Be({"gate": 14336 * 4096, "up": 14336 * 4096}, {"gate": (114688, 224), "up": (114688, 224)})
    f = FusedGemv.__new__(FusedGemv)
    f.manager = Mgr(be)
    f._fit_geometry(group_of(["gate", "up"]), cus=cus)
    assert be.geo["gate"] == (304 * 512, 304)
    # groups too small to fill the device inside the default budget keep what they have
    for sizes in ({"q": 4096 * 4096, "k": 1024 * 4096, "v": 1024 * 4096}, {"a": 3_000_000, "b": 5_000_001}):
        be = Be(sizes, {h: (131072, 256) for h in sizes})
        f = FusedGemv.__new__(FusedGemv)
        f.manager = Mgr(be)
        f._fit_geometry(group_of(list(sizes)), cus=cus)
        assert f.manager.written == [] and all(g == (131072, 256) for g in be.geo.values())


def test_small_blocks_share_a_decode_launch():
    """DecompressAhead merges consecutive blocks until a launch holds enough
    elements to fill the device or 16 tensors (host logic, no GPU)."""
    from neuzip_amd.prefetch import _merge_small

    blocks = [[f"b{i}.{k}" for k in range(4)] for i in range(24)]          # GPT-2-medium: 4 weights, 12.6 M per block
    size = lambda name: {"0": 3145728, "1": 1048576, "2": 4194304, "3": 4194304}[name[-1]]
    merged = _merge_small(blocks, size, 2 * 4 * 256 * 64 * 256)
    assert [len(g) for g in merged] == [12] * 8 and merged[0][:5] == ["b0.0", "b0.1", "b0.2", "b0.3", "b1.0"]
    big = [[f"l{i}.{k}" for k in range(7)] for i in range(4)]               # an 8B block fills the device by itself
    assert _merge_small(big, lambda name: 30_000_000, 2 * 4 * 256 * 64 * 256) == big
    tiny = [[f"t{i}"] for i in range(40)]                                    # never more than 16 tensors per launch
    assert [len(g) for g in _merge_small(tiny, lambda name: 1000, 10 ** 9)] == [16, 16, 8]
