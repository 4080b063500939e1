"""Host logic of the quantization graph rewrite and of the torch.compile hook, on the CPU.

The rules call the package's quantize / dequantize / quantized-matmul operators, which need the GPU; here those three
are replaced by stand-ins computed with the oracle, so that what is tested is the rewriting itself (which nodes match,
what replaces them, which conditions keep the fused operator away), PassContext, and persistence.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from torch import fx

import hidet_amd
from hidet_amd.graph import PassContext, quant as quant_patterns
from hidet_amd.graph.frontend.torch import QuantizedWeightStore, quantize_module
from hidet_amd.graph.ops import quant as quant_ops
from hidet_amd.graph.transforms.graph_patterns.quant import (SymmetricLinearQuantizePatternR, SymmetricQuantizeMatmulFused,
                                                             SymmetricEmbeddingQuantizePattern)
from oracle import oracle as O

_NP = {torch.float32: 'float32', torch.float16: 'float16'}


@pytest.fixture
def cpu_ops(monkeypatch):
    calls = {'quantize': 0, 'dequantize': 0, 'matmul': 0}

    def symmetric_quantize(w, quant_type='int8', dims=-1):
        calls['quantize'] += 1
        q, s = O.symmetric_quantize(w.detach().numpy(), quant_type, dims=dims)
        return torch.from_numpy(q), torch.from_numpy(s)

    def symmetric_dequantize(wq, scale, dims=-1):
        calls['dequantize'] += 1
        return torch.from_numpy(O.symmetric_dequantize(wq.numpy(), scale.numpy(), dims=dims))

    def symmetric_quant_matmul(a, wq, scale, bias=None):
        calls['matmul'] += 1
        assert a.dtype == torch.float16 and wq.dtype == torch.int8 and scale.dtype == torch.float16
        a2 = a.reshape(-1, a.shape[-1]).numpy()
        out = torch.from_numpy(O.symmetric_quant_matmul(a2, wq.numpy(), scale.numpy())).reshape(*a.shape[:-1], wq.shape[1])
        if bias is not None:
            calls['bias'] = calls.get('bias', 0) + 1
            assert bias.dtype == torch.float16 and tuple(bias.shape) == (wq.shape[1],)
            out = out + bias
        return out

    monkeypatch.setattr(quant_ops, 'symmetric_quantize', symmetric_quantize)
    monkeypatch.setattr(quant_ops, 'symmetric_dequantize', symmetric_dequantize)
    monkeypatch.setattr(quant_ops, 'symmetric_quant_matmul', symmetric_quant_matmul)
    return calls


def _targets(gm):
    return [n.target for n in gm.graph.nodes if n.op in ('call_function', 'call_module', 'call_method')]


class Mlp(torch.nn.Module):
    def __init__(self, d=32, h=64, bias=True):
        super().__init__()
        self.up = torch.nn.Linear(d, h, bias=bias)
        self.down = torch.nn.Linear(h, d, bias=bias)

    def forward(self, x):
        return self.down(F.gelu(self.up(x)))


def test_pass_context_mirrors_reference_api():
    with PassContext() as ctx:
        assert PassContext.current() is ctx
        ctx.set_precision('int8')
        assert ctx.configs['precision'] == 'float16'
        names = [type(r).__name__ for r in ctx.configs['quantize_patterns']]
        assert names == ['SymmetricLinearQuantizePatternR', 'SymmetricLinearQuantizePatternL',
                         'SymmetricQuantizeMatmulFused', 'SymmetricEmbeddingQuantizePattern']
        ctx.add_quantize_rules(None)
        assert ctx.configs['quantize_patterns'] == []
        ctx.add_quantize_rules([SymmetricQuantizeMatmulFused, SymmetricLinearQuantizePatternR('int16', dims=0)])
        assert isinstance(ctx.configs['quantize_patterns'][0], SymmetricQuantizeMatmulFused)
        with pytest.raises(TypeError):
            ctx.add_quantize_rules([3])
        with pytest.raises(ValueError):
            ctx.set_precision('int4')
        ctx.set_precision('bfloat16')
        assert ctx.configs['precision'] == 'bfloat16'
    assert PassContext.current() is not ctx
    assert len(quant_patterns.default_patterns()) == 4
    assert len(quant_patterns.symmetric_linear_patterns('int16', dims=0)) == 3
    assert len(quant_patterns.symmetric_embedding_patterns()) == 1


def test_linear_modules_become_fused_operator(cpu_ops):
    torch.manual_seed(0)
    model = Mlp().eval()
    x = torch.randn(3, 5, 32)
    want = model(x)
    with PassContext() as ctx:
        ctx.set_precision('int8')
        gm = quantize_module(model, ctx)
        assert dict(ctx.rewrites)[ctx.configs['quantize_patterns'][0].name] == 2
        assert dict(ctx.rewrites)[ctx.configs['quantize_patterns'][2].name] == 2
    targets = _targets(gm)
    assert targets.count(quant_ops.symmetric_quant_matmul) == 2
    assert quant_ops.symmetric_dequantize not in targets and 'up' not in targets and 'down' not in targets
    assert cpu_ops['quantize'] == 2
    consts = {n: b for n, b in gm.named_buffers()}
    assert consts['up_weight_wq'].dtype == torch.int8 and tuple(consts['up_weight_wq'].shape) == (32, 64)  # [K, N]
    assert consts['up_weight_scale'].dtype == torch.float16 and tuple(consts['up_weight_scale'].shape) == (64,)
    got = gm(x.half())
    assert got.dtype == torch.float16 and cpu_ops['matmul'] == 2
    assert O.max_rel_err(got.float().numpy(), want.detach().numpy()) < 3e-2


def test_bias_moves_into_the_fused_operator(cpu_ops):
    # nn.Linear with bias: matmul + add becomes one call of the fused operator with the bias as its fourth argument
    torch.manual_seed(5)
    model = Mlp(bias=True).eval()
    x = torch.randn(2, 7, 32)
    want = model(x)
    with PassContext() as ctx:
        ctx.set_precision('int8')
        gm = quantize_module(model, ctx)
        assert ctx.rewrites[-1][1] == 2  # the epilogue rule ran last and fused both layers
    targets = _targets(gm)
    assert targets.count(quant_ops.symmetric_quant_matmul) == 2 and torch.add not in targets
    mm_nodes = [n for n in gm.graph.nodes if n.op == 'call_function' and n.target is quant_ops.symmetric_quant_matmul]
    assert all(len(n.args) == 4 for n in mm_nodes)
    got = gm(x.half())
    assert cpu_ops.get('bias') == 2
    assert O.max_rel_err(got.float().numpy(), want.detach().numpy()) < 3e-2
    # without bias nothing changes; a bias that is not a constant vector of N elements stays an add
    with PassContext() as ctx:
        ctx.set_precision('int8')
        gm2 = quantize_module(Mlp(bias=False).eval(), ctx)
        assert ctx.rewrites[-1][1] == 0
    assert all(len(n.args) == 3 for n in gm2.graph.nodes if n.op == 'call_function' and n.target is quant_ops.symmetric_quant_matmul)


def test_quantize_module_leaves_the_source_model_untouched(cpu_ops):
    # the rewrite casts constants to float16 and swaps weights for int8 codes in a copy; the caller's model keeps its
    # float32 parameters, bit for bit
    torch.manual_seed(4)
    model = Mlp().eval()
    before = {k: v.clone() for k, v in model.state_dict().items()}
    with PassContext() as ctx:
        ctx.set_precision('int8')
        quantize_module(model, ctx)
    after = model.state_dict()
    assert set(after) == set(before)
    for k, v in before.items():
        assert after[k].dtype == torch.float32 and torch.equal(after[k], v), k


def test_decode_layout_keeps_codes_k_contiguous_and_releases_the_rest(cpu_ops):
    torch.manual_seed(2)
    model = Mlp().eval()
    x = torch.randn(2, 32)
    want = model(x)
    with PassContext() as ctx:
        ctx.set_precision('int8').set_decode_layout()
        assert ctx.configs['decode_layout'] is True
        gm = quantize_module(model, ctx)
    consts = {n: b for n, b in gm.named_buffers()}
    # one int8 constant per layer, [K, N] with K contiguous; the row-major codes and the float modules are gone
    assert sorted(consts) == ['down_bias', 'down_weight_scale', 'down_weight_wq_kc', 'up_bias', 'up_weight_scale', 'up_weight_wq_kc']
    up = consts['up_weight_wq_kc']
    assert tuple(up.shape) == (32, 64) and up.stride() == (1, 32) and up.dtype == torch.int8
    assert not hasattr(gm, 'up') and not hasattr(gm, 'down')
    q, _ = O.symmetric_quantize(model.up.weight.detach().half().t().contiguous().numpy(), 'int8', dims=0)
    assert np.array_equal(up.numpy(), q)
    got = gm(x.half())
    assert O.max_rel_err(got.float().numpy(), want.detach().numpy()) < 3e-2
    # without the option nothing changes in the constants' layout, and unused float modules are released all the same
    with PassContext() as ctx:
        ctx.set_precision('int8')
        gm2 = quantize_module(Mlp().eval(), ctx)
    assert gm2.up_weight_wq.is_contiguous() and not hasattr(gm2, 'up')


def test_functional_linear_matmul_right_and_left(cpu_ops):
    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.w1 = torch.nn.Parameter(torch.randn(24, 16))   # F.linear weight [out, in]
            self.b1 = torch.nn.Parameter(torch.randn(24))
            self.w2 = torch.nn.Parameter(torch.randn(24, 8))    # x @ w2
            self.w3 = torch.nn.Parameter(torch.randn(4, 6))     # w3 @ y
            self.w4 = torch.nn.Parameter(torch.randn(2, 3, 8))  # not two-dimensional: left alone

        def forward(self, x):
            y = torch.matmul(F.linear(x, self.w1, self.b1), self.w2)     # [6, 8]
            return self.w3 @ y + torch.matmul(y, self.w4.sum(0).t()).sum()

    torch.manual_seed(1)
    model = M().eval()
    x = torch.randn(6, 16)
    want = model(x)
    with PassContext() as ctx:
        ctx.set_precision('int8')
        gm = quantize_module(model, ctx)
    targets = _targets(gm)
    assert targets.count(quant_ops.symmetric_quant_matmul) == 2      # F.linear and x @ w2
    assert targets.count(quant_ops.symmetric_dequantize) == 1        # w3 @ y keeps matmul(dequant(wq, scale), y)
    assert F.linear not in targets
    got = gm(x.half())
    assert O.max_rel_err(got.float().numpy(), want.detach().numpy()) < 5e-2


def test_fused_rule_conditions(cpu_ops):
    def rewritten(model, precision, rules):
        with PassContext() as ctx:
            ctx.set_precision(precision)
            ctx.add_quantize_rules(rules)
            return _targets(quantize_module(model, ctx))

    torch.manual_seed(2)
    # N not a multiple of 4: stays matmul over the dequantized weight
    t = rewritten(torch.nn.Linear(16, 6, bias=False).eval(), 'float16', quant_patterns.symmetric_linear_patterns())
    assert quant_ops.symmetric_quant_matmul not in t and quant_ops.symmetric_dequantize in t
    # int16 codes: not the fused operator's type
    t = rewritten(torch.nn.Linear(16, 8, bias=False).eval(), 'float16', quant_patterns.symmetric_linear_patterns('int16'))
    assert quant_ops.symmetric_quant_matmul not in t and quant_ops.symmetric_dequantize in t
    # float32 model (no precision set): the fused operator is float16 only
    t = rewritten(torch.nn.Linear(16, 8, bias=False).eval(), None, quant_patterns.symmetric_linear_patterns())
    assert quant_ops.symmetric_quant_matmul not in t and quant_ops.symmetric_dequantize in t
    # all conditions met
    t = rewritten(torch.nn.Linear(16, 8, bias=False).eval(), 'float16', quant_patterns.symmetric_linear_patterns())
    assert t.count(quant_ops.symmetric_quant_matmul) == 1 and quant_ops.symmetric_dequantize not in t


def test_embedding_rule(cpu_ops):
    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Embedding(50, 16)
            self.table = torch.nn.Parameter(torch.randn(20, 8))

        def forward(self, ids, ids2):
            return self.emb(ids), F.embedding(ids2, self.table)

    torch.manual_seed(3)
    model = M().eval()
    ids, ids2 = torch.randint(0, 50, (2, 7)), torch.randint(0, 20, (5,))
    want = model(ids, ids2)
    with PassContext() as ctx:
        ctx.add_quantize_rules([SymmetricEmbeddingQuantizePattern()])
        gm = quantize_module(model, ctx)
        assert ctx.rewrites[0][1] == 2
    got = gm(ids, ids2)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        assert O.max_rel_err(g.detach().numpy(), w.detach().numpy()) < 1e-2
    # exactly the oracle's per-row quantization of the table
    q, s = O.symmetric_quantize(model.table.detach().numpy(), 'int8', dims=[-1])
    ref = O.symmetric_dequantize(q, s, dims=[-1])[ids2.numpy()]
    assert np.array_equal(got[1].detach().numpy(), ref)


def test_quantized_weights_persist_and_are_reused(cpu_ops, tmp_path):
    torch.manual_seed(4)
    model = Mlp(bias=False).eval()
    store = QuantizedWeightStore()
    with PassContext() as ctx:
        ctx.set_precision('int8').set_quantized_weights(store)
        gm = quantize_module(model, ctx)
    assert sorted(store) == ['down.weight', 'up.weight'] and cpu_ops['quantize'] == 2
    store['bf16.entry'] = (torch.arange(6, dtype=torch.int8).reshape(2, 3), torch.tensor([0.5, 2.0, 3.0], dtype=torch.bfloat16))
    path = str(tmp_path / 'quantized.npz')
    store.save(path)
    loaded = QuantizedWeightStore.load(path)
    assert sorted(loaded) == sorted(store)
    for name in store:
        assert torch.equal(loaded[name][0], store[name][0]) and loaded[name][0].dtype == store[name][0].dtype
        assert torch.equal(loaded[name][1], store[name][1]) and loaded[name][1].dtype == store[name][1].dtype
    assert loaded.nbytes() == store.nbytes()
    with PassContext() as ctx:
        ctx.set_precision('int8').set_quantized_weights(loaded)
        gm2 = quantize_module(Mlp(bias=False).eval(), ctx)   # different random weights: the stored ones must win
    assert cpu_ops['quantize'] == 2                          # nothing was quantized again
    x = torch.randn(4, 32).half()
    assert torch.equal(gm(x), gm2(x))


def test_torch_compile_backend_is_registered_and_rewrites(cpu_ops):
    from torch._dynamo import list_backends

    assert 'hidet' in list_backends(None)
    torch.manual_seed(5)
    model = Mlp().eval()
    x = torch.randn(4, 32)
    want = model(x)
    torch._dynamo.reset()
    with PassContext() as ctx:
        ctx.set_precision('int8')
        compiled = torch.compile(model, backend='hidet')
        with torch.no_grad():
            got = compiled(x)
        fused = dict(ctx.rewrites).get(ctx.configs['quantize_patterns'][2].name, 0)
    assert fused == 2 and cpu_ops['matmul'] >= 2
    assert got.dtype == torch.float32 and got.shape == want.shape   # cast back to the caller's dtype
    assert O.max_rel_err(got.numpy(), want.detach().numpy()) < 3e-2
