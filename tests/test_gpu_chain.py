"""Layer-chain runner: convolutions back to back on u8 NCHW16c activations, bit-exact against the same
chain composed from the oracle's operators (the requantisation itself is an extension without a
reference counterpart; the convolution inside each layer is the pinned one)."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import chain, rng

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _oracle_chain(oracle, layers_np, x):
    outs = []
    for w, b, scale, shift, stride, pad, source in layers_np:
        src = x if source < 0 else outs[source]
        outs.append(oracle.conv2d_nchwc_u8_requant(src, oracle.prepack_conv_weight(w, 16), b, scale, shift, stride, pad, 1,
                                                   conv=oracle.c_conv2d_nchwc))
    return outs


def _small_layers():
    spec = [  # oc, ic, k, stride, pad, source (None = previous)
        (32, 16, 3, 1, 1, None),
        (32, 32, 1, 2, 0, None),
        (16, 32, 3, 1, 1, None),
        (48, 32, 1, 2, 0, 0),     # side branch on layer 0's output
        (16, 16, 3, 2, (1, 0, 1, 2), 2),
    ]
    out = []
    for i, (oc, ic, k, stride, pad, source) in enumerate(spec):
        w = rng.uniform_s8((oc, ic, k, k), 100 + i)
        b = rng.uniform_s8((oc,), 200 + i).astype(np.int32) * 1000 if i % 2 == 0 else None
        out.append((w, b, 3 + i, 13, stride, pad, i - 1 if source is None else source))
    return out


def _to_chain(layers_np, dev):
    return [chain.ChainLayer(_t(w, dev), None if b is None else _t(b, dev), scale, shift, stride, pad, source)
            for w, b, scale, shift, stride, pad, source in layers_np]


def test_chain_with_side_branch_bit_exact(dev, oracle):
    layers_np = _small_layers()
    x = rng.uniform_u8((3, 1, 13, 11, 16), 7)
    want = _oracle_chain(oracle, layers_np, x)
    c = chain.ConvChain(_to_chain(layers_np, dev), x.shape)
    last = c(_t(x, dev))
    torch.cuda.synchronize()
    for i, w in enumerate(want):
        got = c.outputs[i].cpu().numpy()
        assert got.shape == w.shape and np.array_equal(got, w), f"layer {i} ({c.variants[i]})"
        assert 0 < w.max() and (w > 0).mean() > 0.05, "degenerate case: the requantised activations are all zero"
    assert last is c.outputs[-1]


def test_chain_graph_replay_follows_the_input(dev, oracle):
    layers_np = _small_layers()[:3]
    x1 = rng.uniform_u8((2, 1, 9, 9, 16), 8)
    x2 = rng.uniform_u8((2, 1, 9, 9, 16), 9)
    c = chain.ConvChain(_to_chain(layers_np, dev), x1.shape)
    xd = _t(x1, dev)
    replay = c.graph(xd)
    for x in (x1, x2, x1):  # the program's own eager work and synchronisations between the replays
        xd.copy_(_t(x, dev))
        torch.cuda.synchronize()
        got = replay().cpu().numpy()
        assert np.array_equal(got, _oracle_chain(oracle, layers_np, x)[-1])


@pytest.mark.parametrize("builder,count,last_shape", [(chain.resnet50_layers, 52, (1, 128, 7, 7, 16)),
                                                      (chain.resnet18_layers, 19, (1, 32, 7, 7, 16))])
def test_resnet_chain_batch1_bit_exact(dev, oracle, builder, count, last_shape):
    """Every layer at batch 1.  The oracle runs first, layer by layer, and picks each layer's shift from its own
    int32 sums (95th percentile -> about 200) so that the activations stay spread over 0..255 down the chain."""
    weights = []

    def make_weight(oc, ic, k):
        weights.append(rng.uniform_s8((oc, ic, k, k), 1000 + len(weights)))
        return _t(weights[-1], dev)

    layers = builder(make_weight)
    assert len(layers) == count
    x = rng.uniform_u8((1, 4, 56, 56, 16), 5)
    want = []
    for i, ly in enumerate(layers):
        src = x if ly.source < 0 else want[ly.source]
        wp = oracle.prepack_conv_weight(weights[i], 16)
        acc = oracle.c_conv2d_nchwc(src, wp, ly.stride, ly.padding, 1)
        shift = max(1, int(np.ceil(np.log2(max(np.percentile(acc, 95), 1.0) * 3 / 200))))
        layers[i] = ly._replace(scale=3, shift=shift)
        want.append(oracle.conv2d_nchwc_u8_requant(src, wp, None, 3, shift, ly.stride, ly.padding, 1,
                                                   conv=lambda *a, **k: acc))
    c = chain.ConvChain(layers, x.shape)
    c(_t(x, dev))
    torch.cuda.synchronize()
    for i, w in enumerate(want):
        assert np.array_equal(c.outputs[i].cpu().numpy(), w), f"layer {i} ({c.variants[i]})"
        assert (w > 0).mean() > 0.2 and w.max() > 100, f"layer {i}: degenerate activations"
    assert tuple(c.outputs[-1].shape) == last_shape


def test_chain_rejects_mismatched_layers(dev):
    w = torch.zeros((32, 16, 1, 1), dtype=torch.int8, device=dev)
    with pytest.raises(ValueError, match="channels"):
        chain.ConvChain([chain.ChainLayer(w, None, 1, 8, 1, 0)], (1, 2, 4, 4, 16))
    with pytest.raises(ValueError, match="earlier layer"):
        chain.ConvChain([chain.ChainLayer(w, None, 1, 8, 1, 0, 0)], (1, 1, 4, 4, 16))
    with pytest.raises(ValueError, match="shift"):
        chain.ConvChain([chain.ChainLayer(w, None, 1, 0, 1, 0)], (1, 1, 4, 4, 16))
    c = chain.ConvChain([chain.ChainLayer(w, None, 1, 8, 1, 0)], (1, 1, 4, 4, 16))
    with pytest.raises(ValueError, match="expected"):
        c(torch.zeros((1, 1, 5, 4, 16), dtype=torch.uint8, device=dev))
