"""The quantization graph rewrite and `torch.compile(backend='hidet')` on the GPU: linear layers of a small
transformer-style model run on the HIP W8A16 kernels, embeddings on the int8 table. Semantics of the reference's
tests/models/test_quant_gpt2.py (quantized logits vs float logits, atol = rtol = 0.5), with a tighter bound here."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import hidet_amd
from hidet_amd.graph import PassContext
from hidet_amd.graph.frontend.torch import QuantizedWeightStore, quantize_module
from hidet_amd.graph.ops import quant as quant_ops
from oracle import oracle as O
from gpu_util import announce

pytestmark = pytest.mark.gpu


class Block(torch.nn.Module):
    def __init__(self, d, heads):
        super().__init__()
        self.heads = heads
        self.ln1, self.ln2 = torch.nn.LayerNorm(d), torch.nn.LayerNorm(d)
        self.qkv, self.proj = torch.nn.Linear(d, 3 * d), torch.nn.Linear(d, d)
        self.up, self.down = torch.nn.Linear(d, 4 * d), torch.nn.Linear(4 * d, d)

    def forward(self, x):
        b, t, d = x.shape
        q, k, v = self.qkv(self.ln1(x)).view(b, t, 3, self.heads, d // self.heads).permute(2, 0, 3, 1, 4)
        att = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(b, t, d)
        x = x + self.proj(att)
        return x + self.down(F.gelu(self.up(self.ln2(x))))


class TinyGpt(torch.nn.Module):
    def __init__(self, vocab=512, d=256, heads=4, layers=2, ctx=64):
        super().__init__()
        self.wte, self.wpe = torch.nn.Embedding(vocab, d), torch.nn.Embedding(ctx, d)
        self.blocks = torch.nn.ModuleList(Block(d, heads) for _ in range(layers))
        self.ln_f = torch.nn.LayerNorm(d)
        self.head = torch.nn.Linear(d, vocab, bias=False)

    def forward(self, ids):
        pos = torch.arange(ids.shape[1], device=ids.device)
        x = self.wte(ids) + self.wpe(pos)
        for blk in self.blocks:
            x = blk(x)
        return self.head(self.ln_f(x))


def _graph_targets(gm):
    return [n.target for n in gm.graph.nodes if n.op == 'call_function']


def test_torch_compile_int8_runs_linears_on_hip_kernels():
    announce('graph rewrite: torch.compile backend=hidet, int8')
    torch.manual_seed(0)
    model = TinyGpt().cuda().eval()
    ids = torch.randint(0, 512, (2, 48), device='cuda')
    with torch.no_grad():
        want = model(ids)
    torch._dynamo.reset()
    with PassContext() as ctx:
        ctx.set_precision('int8')
        compiled = torch.compile(model, backend='hidet')
        with torch.no_grad():
            got = compiled(ids)
            again = compiled(ids)
        counts = dict(ctx.rewrites)
    rules = hidet_amd.graph.quant.default_patterns()
    assert counts[rules[0].name] == 9            # 4 linears per block x 2 + the head
    assert counts[rules[2].name] == 9            # all of them meet the fused operator's conditions
    assert counts[rules[3].name] == 2            # both embedding tables
    assert got.dtype == want.dtype and got.shape == want.shape
    assert torch.equal(got, again)
    err = O.max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy())
    print('max_rel_err of int8 logits vs float32 logits', err)
    assert err < 5e-2
    assert torch.allclose(got, want, atol=0.5, rtol=0.5)   # the reference's own bound


def test_ahead_of_time_rewrite_and_persisted_weights(tmp_path):
    announce('graph rewrite: quantize_module + persisted weights')
    torch.manual_seed(1)

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up, self.down = torch.nn.Linear(512, 1024), torch.nn.Linear(1024, 512, bias=False)

        def forward(self, x):
            return self.down(F.gelu(self.up(x)))

    model = Mlp().cuda().eval()
    x = torch.randn(3, 40, 512, device='cuda')
    with torch.no_grad():
        want = model(x)
    store = QuantizedWeightStore()
    with PassContext() as ctx:
        ctx.set_precision('int8').set_quantized_weights(store)
        gm = quantize_module(model, ctx)
    targets = _graph_targets(gm)
    assert targets.count(quant_ops.symmetric_quant_matmul) == 2 and quant_ops.symmetric_dequantize not in targets
    with torch.no_grad():
        got = gm(x.half())
    assert O.max_rel_err(got.float().cpu().numpy(), want.cpu().numpy()) < 3e-2
    # the stored codes are what the oracle computes from the float16 weights, bit for bit
    w_kn = model.up.weight.detach().half().t().contiguous().cpu().numpy()
    q, s = O.symmetric_quantize(w_kn, 'int8', dims=0, target='gpu')
    assert np.array_equal(store['up.weight'][0].cpu().numpy(), q) and np.array_equal(store['up.weight'][1].cpu().numpy(), s)
    # save, load, rebuild from the stored weights only
    path = str(tmp_path / 'mlp_int8.npz')
    store.save(path)
    loaded = QuantizedWeightStore.load(path, device='cuda')
    blank = Mlp().cuda().eval()
    with torch.no_grad():
        blank.up.bias.copy_(model.up.bias)       # biases are not quantized; the weights come from the store
    with PassContext() as ctx:
        ctx.set_precision('int8').set_quantized_weights(loaded)
        gm2 = quantize_module(blank, ctx)
    with torch.no_grad():
        assert torch.equal(gm2(x.half()), got)


def test_decode_layout_runs_decode_and_prefill_calls():
    announce('graph rewrite: decode layout')
    torch.manual_seed(3)

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up, self.down = torch.nn.Linear(512, 1024), torch.nn.Linear(1024, 512, bias=False)

        def forward(self, x):
            return self.down(F.gelu(self.up(x)))

    model = Mlp().cuda().eval()
    with PassContext() as ctx:
        ctx.set_precision('int8')
        plain = quantize_module(model, ctx)
    with PassContext() as ctx:
        ctx.set_precision('int8').set_decode_layout()
        gm = quantize_module(model, ctx)
    assert gm.up_weight_wq_kc.stride() == (1, 512) and torch.equal(gm.up_weight_wq_kc, plain.up_weight_wq)
    for rows in (1, 3, 40, 100, 16, 1):  # decode-sized calls, batched decode (the GEMM on the same layout), a prefill-sized one
                                         # (row-major copy made once), decode again
        x = torch.randn(rows, 512, device='cuda', dtype=torch.float16)
        with torch.no_grad():
            got, want = gm(x), plain(x)
        assert got.shape == want.shape
        assert O.max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy()) < 2e-3
    from hidet_amd.graph.ops.quant import matmul as qmm
    entry = qmm._ROW_MAJOR_COPIES.get(gm.up_weight_wq_kc)
    assert entry is not None and entry[1].is_contiguous() and torch.equal(entry[1], gm.up_weight_wq_kc)
    # a weight written in place gets a fresh copy on the next prefill-sized call
    gm.up_weight_wq_kc.zero_()
    x = torch.randn(100, 512, device='cuda', dtype=torch.float16)
    with torch.no_grad():
        gm(x)
    assert int(qmm._ROW_MAJOR_COPIES.get(gm.up_weight_wq_kc)[1].abs().sum()) == 0
