"""Parity of the full-size benchmark workloads (C2, C3, C4, and layers 0 and 7 + head of the packed C5) with the CPU oracle, run on the host cores of the GPU box
on the same weights, token ids and labels.  The comparison rule (stated bar against the fp32 oracle; where a chain of
bf16-stored ops cannot meet it, no farther from fp32 than the oracle's exact-arithmetic bf16-storage evaluation) is in
tests/_parity.py.

1. Layer by layer (all three workloads).  The HIP step records the bf16 input and output of every decoder layer and the
   gradients that arrive at them.  The fp32 oracle then re-evaluates each layer from the very input the HIP layer saw
   and back-propagates the very output gradient the HIP layer received: layer output, input gradient and every weight
   gradient of that layer are compared, and so are the final norm + LM head + loss (logits, loss, gradients) from the
   last hidden state, and the embedding gradient from the first layer's input gradient.  Every parameter gradient of the
   model is covered, each against fp32 arithmetic on identical inputs.  Layers 1.. and the head meet the stated bar as
   they are; layer 0, whose input is the small-norm embedding so that its output is all its own update, sits at the
   bf16-storage floor of one layer (about 1.1 - 1.5 % relative L2 at these widths).

2. End to end (C2, the headline workload): loss at 1e-3; logits and every gradient against the fp32 oracle and the
   bf16-storage oracle run on the whole stack.
"""
import time

import pytest
import torch

import _parity as P
from oracle import llama_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


def _oracle_cfg(w):
    return dict(num_layers=w["num_layers"], hidden_size=w["hidden_size"], num_attention_heads=w["num_attention_heads"],
                num_kv_attention_heads=w["num_kv_attention_heads"], head_dim=w["hidden_size"] // w["num_attention_heads"],
                intermediate_size=w["intermediate_size"], vocab_size=w["vocab_size"])


def _hip_step(name, dev):
    """Runs the workload's step on the GPU and returns everything the comparisons need, on the host."""
    from easyllm_amd import runner, workloads as W
    from easyllm_amd.transformer import ParallelTransformerLayerPipe
    w = dict(W.WORKLOADS[name])
    torch.manual_seed(w["seed"])
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w)})
    with torch.no_grad():  # norm weights away from 1 so that their gradients carry information
        g = torch.Generator().manual_seed(w["seed"])
        for n, p in model.named_parameters():
            if p.dim() == 1:
                p.copy_((1.0 + 0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
    runner.attach_main_grads(model)
    inputs, (labels, loss_mask), _ = W.make_inputs(w)
    rec = {"x": {}, "dy": {}, "dx": {}}
    hooks = []

    def hook_layer(idx):
        def fwd(module, args, out):
            x_in = args[0][0] if isinstance(args[0], (tuple, list)) else args[0]
            x_out = out[0] if isinstance(out, (tuple, list)) else out
            # a layer under activation checkpointing runs twice: first without a graph (nothing to hook), then again
            # inside backward, where its output receives the gradient
            rec["x"][idx] = x_in.detach()
            rec["x"][idx + 1] = x_out.detach()
            if x_out.requires_grad:
                x_out.register_hook(lambda gr: rec["dy"].__setitem__(idx, gr.detach().clone()))
            if x_in.requires_grad:
                x_in.register_hook(lambda gr: rec["dx"].__setitem__(idx, gr.detach().clone()))
        return fwd

    layers = [(n, m) for n, m in model.named_children() if isinstance(m, ParallelTransformerLayerPipe)]
    assert len(layers) == w["num_layers"]
    for i, (n, m) in enumerate(layers):
        hooks.append(m.register_forward_hook(hook_layer(i)))
    to_dev = lambda t: tuple(None if x is None else x.to(dev) for x in t)  # noqa: E731
    logits = model(to_dev(inputs))
    logits_host = logits.detach().float().cpu()
    loss = model.loss_fn(logits, (labels.to(dev), loss_mask.to(dev)))
    loss.backward()
    torch.cuda.synchronize()
    for hk in hooks:
        hk.remove()
    out = dict(w=w, tokens=inputs[0], labels=labels, loss_mask=loss_mask, logits=logits_host, loss=loss.item(),
               position_ids=inputs[1] if len(inputs) > 3 else None, cu_seqlens=inputs[3] if len(inputs) > 3 else None,
               recomputed=model.recompute_count,
               grads={n: p.main_grad.cpu() for n, p in model.named_parameters()},
               W={k: v.detach().float().cpu() for k, v in model.state_dict().items() if "inv_freq" not in k},
               x={i: t.float().cpu() for i, t in rec["x"].items()},
               dy={i: t.float().cpu() for i, t in rec["dy"].items()},
               dx={i: t.float().cpu() for i, t in rec["dx"].items()})
    del model, logits, loss, rec
    torch.cuda.empty_cache()
    return out


def _layer_eval(r, cfg, i, storage):
    """Oracle evaluation of decoder layer i from the HIP layer's own input and output gradient."""
    p = O.layer_prefix(i)
    Wl = {k: v.clone().requires_grad_(True) for k, v in r["W"].items() if k.startswith(p)}
    x = r["x"][i].clone().requires_grad_(True)
    out = O.decoder_layer(x, Wl, p, cfg, position_ids=r["position_ids"], cu_seqlens=r["cu_seqlens"], storage_dtype=storage)
    out.backward(r["dy"][i])
    res = {"out": out.detach(), "dx": x.grad}
    res.update({k: v.grad for k, v in Wl.items()})
    return res


class _Lazy:
    def __init__(self, fn):
        self.fn, self.value = fn, None

    def item(self, key):
        def get():
            if self.value is None:
                self.value = self.fn()
            return self.value[key]
        return get


def _layer_by_layer(name, r, only=None):
    """Part 1 of the module docstring.  only: the decoder layers to evaluate (default all)."""
    w, Wt, cfg = r["w"], r["W"], _oracle_cfg(r["w"])
    L = w["num_layers"]
    rep = P.Report(name)
    for i in (range(L) if only is None else only):
        ref = _layer_eval(r, cfg, i, None)
        floor = _Lazy(lambda i=i: _layer_eval(r, cfg, i, torch.bfloat16))
        rep.check("layer %d output" % i, r["x"][i + 1], ref["out"], floor.item("out"))
        rep.check("layer %d input gradient" % i, r["dx"][i], ref["dx"], floor.item("dx"))
        for k in sorted(k for k in ref if k not in ("out", "dx")):
            rep.check("grad " + k, r["grads"][k], ref[k], floor.item(k))
        del ref, floor
    # final norm + untied head + loss from the last hidden state the HIP path produced
    kn, kh = "%d.weight" % (L + 4), "%d.word_embeddings.weight" % (L + 5)
    wn, wh = Wt[kn].clone().requires_grad_(True), Wt[kh].clone().requires_grad_(True)
    xl = r["x"][L].clone().requires_grad_(True)
    logits = O.linear(O.rmsnorm(xl.transpose(0, 1), wn, cfg.get("eps", 1e-6)), wh)
    rep.check("logits from the last hidden state", r["logits"], logits)
    loss = O.cross_entropy_loss(logits, r["labels"], r["loss_mask"])
    rel = abs(r["loss"] - loss.item()) / abs(loss.item())
    rep.note("loss %.6f, oracle from the last hidden state %.6f (rel %.2e)" % (r["loss"], loss.item(), rel), failed=rel > 1e-3)
    loss.backward()
    rep.check("last hidden state gradient", r["dy"][L - 1], xl.grad)
    rep.check("grad " + kn, r["grads"][kn], wn.grad)
    rep.check("grad " + kh, r["grads"][kh], wh.grad)
    # embedding gradient from the gradient that reached the first layer's input ([s, b, h] -> rows in (b s) order)
    ke = "1.word_embeddings.weight"
    ge = O.embedding_bwd(r["tokens"], r["dx"][0].transpose(0, 1), w["vocab_size"])
    rep.check("grad " + ke, r["grads"][ke], ge)
    if only is None:
        assert len([ln for ln in rep.lines if " grad " in ln]) == len(r["grads"])  # every parameter was compared
    return rep


def _oracle_step(Wt, w, tokens, labels, loss_mask, storage):
    Wg = {k: v.clone().requires_grad_(True) for k, v in Wt.items()}
    logits = O.model_forward(Wg, _oracle_cfg(w), tokens, storage_dtype=storage)
    loss = O.cross_entropy_loss(logits, labels, loss_mask)
    loss.backward()
    return logits.detach(), loss.item(), {k: v.grad for k, v in Wg.items()}


@pytest.mark.parametrize("name", ["C2", "C3", "C4"])
def test_every_layer_of_the_full_size_step(gpu_device, name):
    print("full-size parity, layer by layer, workload", name, flush=True)
    r = _hip_step(name, gpu_device)
    t0 = time.time()
    rep = _layer_by_layer(name, r)
    print("\n".join(rep.lines), flush=True)
    print("%s: oracle, layer by layer: %.0f s on the host; %d of %d tensors at the bf16-storage floor, the rest at the "
          "stated bar" % (name, time.time() - t0, rep.floor_used, len(rep.lines) - 1), flush=True)
    assert not rep.failures, "\n".join(rep.failures)
    # only the first layer (embedding-scale input) may need the floor rule
    assert all(" layer 0 " in ln or " grad 3." in ln for ln in rep.lines if "floor]" in ln)


def test_first_and_last_layer_of_the_packed_workload(gpu_device):
    """C5 at its own size (8 layers, 16384 packed tokens in 23 documents, position ids restarting per document, the first 4
    layers recomputed in backward): decoder layers 0 (recomputed) and 7 (not), the final norm + head + loss and the embedding
    gradient, each against the fp32 oracle evaluated from the HIP layer's own input and output gradient -- the packed
    attention forward and backward at 32 heads and the per-document rotary positions at full size."""
    name = "C5"
    print("full-size parity, layers 0 and 7 + head, workload", name, flush=True)
    r = _hip_step(name, gpu_device)
    assert r["recomputed"] == 4 and r["cu_seqlens"] is not None and r["cu_seqlens"].numel() > 3
    t0 = time.time()
    rep = _layer_by_layer(name, r, only=(0, 7))
    print("\n".join(rep.lines), flush=True)
    print("%s: oracle, layers 0 and 7 + head: %.0f s on the host; %d of %d tensors at the bf16-storage floor, the rest at the "
          "stated bar" % (name, time.time() - t0, rep.floor_used, len(rep.lines) - 1), flush=True)
    assert not rep.failures, "\n".join(rep.failures)
    assert all(" layer 0 " in ln or " grad 3." in ln for ln in rep.lines if "floor]" in ln)


# Tensors of the end-to-end comparison that may use the floor rule: all of them -- the error of a four-layer chain of
# bf16-stored ops is past the stated bar for the logits and for every gradient (the layer-by-layer test above is the gate
# that holds each layer to the stated bar on identical inputs) -- but each within 5 % / 25 % of the floor.
def test_headline_workload_end_to_end(gpu_device):
    name = "C2"
    print("full-size parity, end to end, workload", name, flush=True)
    r = _hip_step(name, gpu_device)
    w = r["w"]
    t0 = time.time()
    f_logits, f_loss, f_grads = _oracle_step(r["W"], w, r["tokens"], r["labels"], r["loss_mask"], None)
    s_logits, s_loss, s_grads = _oracle_step(r["W"], w, r["tokens"], r["labels"], r["loss_mask"], torch.bfloat16)
    print("%s: fp32 and bf16-storage oracle steps: %.0f s on the host" % (name, time.time() - t0), flush=True)
    rep = P.Report(name)
    rep.note("loss: HIP %.6f, fp32 oracle %.6f, bf16-storage oracle %.6f" % (r["loss"], f_loss, s_loss),
             failed=abs(r["loss"] - f_loss) > 1e-3 * abs(f_loss))
    rep.check("logits", r["logits"], f_logits, s_logits)
    g = P.gap(r["logits"], s_logits)
    rep.note("logits, HIP vs bf16-storage oracle: max-rel %.2e cosine %.6f L2 %.2e" % g)
    for k in sorted(r["grads"]):
        rep.check("grad " + k, r["grads"][k], f_grads[k], s_grads[k])
    print("\n".join(rep.lines), flush=True)
    assert not rep.failures, "\n".join(rep.failures)
