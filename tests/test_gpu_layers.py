"""Whole layers under the Controller's hooks, compared with the same layer run uncompressed.

The cases and tolerances are those of tests/test_bert.py of the reference (batch norm at L1, layer norm and
the transformer layers at L1.1: outputs equal, gradients within atol 1e-2 / 1e-1, rtol 1e-2).  The reference
builds its transformer layers from the downloaded bert-base-uncased configuration; a default BertConfig has
the same dimensions (768 hidden, 12 heads, 3072 intermediate) and needs no download.  Weights are random in
both: the comparison is between two runs of one layer, not against a trained model.
"""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

import gact
from gact.conf import config as gact_config

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _restore_config():
    saved = copy.copy(gact_config.__dict__)
    yield
    gact_config.__dict__.update(saved)


def forward_backward(layer, data_np, hooks=None, upstream_seed=None):
    """(output, grad wrt input, parameter grads) of one pass; the upstream gradient is all ones as in the
    reference's tests, or seeded normal noise (the gradient of a sum through a final layer norm is zero up to
    rounding, which leaves nothing to compare)."""
    torch.manual_seed(0)
    data = torch.tensor(data_np, device="cuda").requires_grad_()
    layer.zero_grad(set_to_none=True)

    def run():
        out = layer(data)
        out = out[0] if isinstance(out, (tuple, list)) else out
        if upstream_seed is None:
            head = torch.ones_like(out)
        else:
            head = torch.randn(out.shape, generator=torch.Generator().manual_seed(upstream_seed)).to(out.device)
        out.backward(head)
        return out

    if hooks is None:
        out = run()
    else:
        with torch.autograd.graph.saved_tensors_hooks(*hooks):
            out = run()
    grads = [p.grad.detach().cpu().numpy() for p in layer.parameters()]
    return out.detach().cpu().numpy(), data.grad.detach().cpu().numpy(), grads


def compressed_twin(layer, level):
    """A copy of the layer with its own Controller at the given optimisation level."""
    twin = copy.deepcopy(layer)
    gact.set_optimization_level(level)
    controller = gact.controller.Controller(twin)
    return twin, controller, (controller.quantize, controller.dequantize)


def test_batchnorm_under_4_bit_hooks():
    rng = np.random.default_rng(0)
    data = rng.standard_normal((64, 3, 56, 56)).astype(np.float32)
    layer = nn.BatchNorm2d(3).cuda()
    out, grad, (_, g_bias) = forward_backward(layer, data)
    twin, controller, hooks = compressed_twin(layer, "L1")
    out_q, grad_q, (_, g_bias_q) = forward_backward(twin, data, hooks)
    assert controller.quantizer.tid > 0                      # something was compressed
    np.testing.assert_array_equal(out, out_q)                # the forward pass does not see the hooks
    np.testing.assert_allclose(grad, grad_q, atol=1e-2, rtol=1e-2)
    np.testing.assert_allclose(g_bias, g_bias_q, atol=1e-2, rtol=1e-2)


def test_layernorm_under_8_bit_hooks():
    rng = np.random.default_rng(0)
    data = rng.standard_normal((1, 10, 10)).astype(np.float32)
    layer = nn.LayerNorm(10, eps=0).cuda()
    out, grad, (g_w, g_b) = forward_backward(layer, data)
    twin, controller, hooks = compressed_twin(layer, "L1.1")
    out_q, grad_q, (g_w_q, g_b_q) = forward_backward(twin, data, hooks)
    assert controller.quantizer.tid > 0
    np.testing.assert_array_equal(out, out_q)
    np.testing.assert_allclose(grad, grad_q, atol=1e-1, rtol=1e-2)
    np.testing.assert_allclose(g_w, g_w_q, atol=1e-1, rtol=1e-2)
    np.testing.assert_allclose(g_b, g_b_q, atol=1e-1, rtol=1e-2)


def _bert_config():
    transformers = pytest.importorskip("transformers")
    cfg = transformers.BertConfig()          # the dimensions of bert-base-uncased
    cfg.hidden_dropout_prob = 0.0
    cfg.attention_probs_dropout_prob = 0.0
    cfg._attn_implementation = "eager"       # matmul - softmax - matmul, whose saved tensors the hooks see
    return cfg


@pytest.mark.parametrize("which", ["self_attention", "layer"])
def test_transformer_layer_under_8_bit_hooks(which):
    cfg = _bert_config()
    from transformers.models.bert import modeling_bert
    torch.manual_seed(0)
    layer = (modeling_bert.BertSelfAttention(cfg) if which == "self_attention" else modeling_bert.BertLayer(cfg)).cuda()
    rng = np.random.default_rng(1)
    data = rng.standard_normal((8, 512, 768)).astype(np.float32)
    out, grad, _ = forward_backward(layer, data, upstream_seed=7)
    twin, controller, hooks = compressed_twin(layer, "L1.1")
    out_q, grad_q, _ = forward_backward(twin, data, hooks, upstream_seed=7)
    assert controller.quantizer.tid >= (3 if which == "self_attention" else 8)
    np.testing.assert_allclose(out, out_q, atol=1e-1, rtol=1e-2)
    np.testing.assert_allclose(grad, grad_q, atol=1e-1, rtol=1e-2)
    # and the compressed gradient is a good estimate, not merely within the loose bound
    rel = np.linalg.norm(grad - grad_q) / np.linalg.norm(grad)
    assert rel < 0.05, rel


def test_small_bert_trains_under_auto_precision_with_dropout():
    """A small BERT classifier with dropout on, six optimizer steps at L2 (auto precision, 4 bit average) with
    the sensitivities re-measured every three steps: whatever the model saves for backward (float activations,
    dropout masks, integer tensors) passes through the hooks, and the losses follow the uncompressed run."""
    transformers = pytest.importorskip("transformers")
    cfg = transformers.BertConfig(hidden_size=128, num_hidden_layers=2, num_attention_heads=4, intermediate_size=512,
                                  vocab_size=1000, max_position_embeddings=64)
    cfg._attn_implementation = "eager"
    ids = torch.randint(0, 1000, (16, 64), generator=torch.Generator().manual_seed(3)).cuda()
    labels = torch.randint(0, 2, (16,), generator=torch.Generator().manual_seed(4)).cuda()

    def train(level):
        torch.manual_seed(11)
        torch.cuda.manual_seed_all(11)
        model = transformers.BertForSequenceClassification(cfg).cuda().train()
        opt = torch.optim.SGD(model.parameters(), lr=0.05)
        controller = None
        if level is not None:
            gact.set_optimization_level(level)
            gact_config.adapt_interval = 3
            controller = gact.controller.Controller(model)
            controller.install_hook()
        losses = []
        try:
            for step in range(6):
                def backprop():
                    torch.manual_seed(100 + step)            # the same dropout masks in both runs and in every probe
                    torch.cuda.manual_seed_all(100 + step)
                    model.zero_grad(set_to_none=True)
                    loss = model(input_ids=ids, labels=labels).loss
                    loss.backward()
                    return loss
                loss = backprop()
                opt.step()
                losses.append(loss.item())
                if controller is not None:
                    controller.iterate(backprop)
        finally:
            if controller is not None:
                controller.uninstall_hook()
        return losses, controller

    exact, _ = train(None)
    compressed, controller = train("L2")
    assert len(controller.quantizer.bits) > 10
    assert set(controller.quantizer.bits.values()) <= {1, 2, 4, 8, 32}
    total = sum(controller.quantizer.dims.values())
    spent = sum(controller.quantizer.bits[t] * controller.quantizer.dims[t] for t in controller.quantizer.bits)
    assert spent <= 4 * total                                # the 4-bit average budget holds
    np.testing.assert_allclose(compressed, exact, atol=0.05)
    assert exact[-1] < exact[0]
