"""Step driver: forward -> loss -> backward for one micro-batch, with fp32 main-grad buffers.

Counterpart of `BaseRunner.forward_step` -> DeepSpeed `train_batch` (llm/runners/base_llm_runner.py:236-245)
for what lies inside this build: `loss = loss_fn(model(inputs), labels); loss.backward()`, weight
gradients landing in fp32 `main_grad` buffers (DeepSpeed's bf16 optimizer accumulates in fp32).
The optimizer step with global-norm clipping that follows lives in optimizer.py; loss scaling by the
number of accumulation steps and ZeRO partitioning are DeepSpeed's and are not reproduced.
"""
import torch

from .registry import MODULE_ZOO_REGISTRY
from . import llama as _llama  # noqa: F401  (registers the model builders)


def build_model(cfg):
    """cfg = {'type': 'llama_custom' | 'llama2_7b' | ..., 'kwargs': {...}} as in the reference's yaml `model:` node."""
    return MODULE_ZOO_REGISTRY.build(cfg)


def attach_main_grads(model):
    """One fp32 gradient buffer per parameter; marks them fresh (first write overwrites)."""
    for p in model.parameters():
        if p.requires_grad:
            p.main_grad = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
            p.main_grad_fresh = True


def zero_main_grads(model):
    """zero_grad without a memset: the next gradient written to each buffer overwrites it."""
    for p in model.parameters():
        if getattr(p, "main_grad", None) is not None:
            p.main_grad_fresh = True
        p.grad = None


def forward_step(model, inputs, labels):
    """One micro-batch: returns the loss tensor after backward has run."""
    output = model(inputs)
    loss = model.loss_fn(output, labels)
    loss.backward()
    return loss


def _tree_map(fn, x):
    if isinstance(x, torch.Tensor):
        return fn(x)
    if isinstance(x, (tuple, list)):
        return type(x)(_tree_map(fn, v) for v in x)
    return x


def _tree_copy(dst, src):
    if isinstance(dst, torch.Tensor):
        dst.copy_(src, non_blocking=True)
    elif isinstance(dst, (tuple, list)):
        for d, s_ in zip(dst, src):
            _tree_copy(d, s_)


class GraphedStep:
    """forward + loss + backward of one micro-batch captured once into a HIP graph and replayed.

    The captured kernels are exactly those of `forward_step`; replaying them removes the per-kernel host work and the
    launch gaps (about 180 launches per step for a 4-layer stack).  Shapes, document boundaries, the checkpoint plan and
    the gradient mode (first micro-batch overwrites `main_grad`, `accumulate=True` adds to it) are frozen at capture
    time; new token ids / labels of the same shape are copied into the static input buffers by `__call__`.  The loss is
    returned as a device tensor that the next replay overwrites.  The token-id range check of the embedding cannot
    raise inside a graph: its flag is read back after every replay and raised one call late, as in the deferred mode.
    """

    def __init__(self, model, inputs, labels, accumulate=False, warmup=2):
        from . import functional
        self.model = model
        self.inputs = _tree_map(lambda t: t.clone(), inputs)
        self.labels = _tree_map(lambda t: t.clone(), labels)
        self._accumulate = accumulate
        self._pending_flag = None

        grads = [p for p in model.parameters() if getattr(p, "main_grad", None) is not None]
        # The eager warm-up passes of an accumulating capture add the capture batch's gradients to the buffers; keep what
        # the buffers (and their "fresh" marks) held and put it back once the graph exists.
        saved = [(p.main_grad.clone(), getattr(p, "main_grad_fresh", False)) for p in grads] if accumulate else None

        def one_step():
            if accumulate:
                for p in grads:  # every captured gradient kernel must add: no buffer may be marked fresh here
                    p.main_grad_fresh = False
            else:
                zero_main_grads(model)
            return forward_step(model, self.inputs, self.labels)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                one_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for p in model.parameters():
            p.grad = None
        del functional.CAPTURED_ID_FLAGS[:]
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.loss = one_step()
        self._flags = list(functional.CAPTURED_ID_FLAGS)
        del functional.CAPTURED_ID_FLAGS[:]
        if saved is not None:
            torch.cuda.synchronize()
            for p, (buf, fresh) in zip(grads, saved):
                p.main_grad.copy_(buf)
                p.main_grad_fresh = fresh
        self._grads = grads
        self._host_flags = [torch.zeros(1, dtype=torch.int32, pin_memory=True) for _ in self._flags]
        self._flag_event = None

    def _check_previous(self):
        from . import functional
        if self._flag_event is not None:
            self._flag_event.synchronize()
            self._flag_event = None
            for host, (_, n) in zip(self._host_flags, self._flags):
                functional._raise_for_id_flag(int(host.item()), self.inputs[0] if isinstance(self.inputs, (tuple, list)) else self.inputs, n)

    def __call__(self, inputs=None, labels=None):
        self._check_previous()
        if inputs is not None:
            _tree_copy(self.inputs, inputs)
        if labels is not None:
            _tree_copy(self.labels, labels)
        if self._accumulate:
            for p in self._grads:  # the graph adds: a buffer marked fresh (zero_main_grads) starts from zero
                if getattr(p, "main_grad_fresh", False):
                    p.main_grad.zero_()
                    p.main_grad_fresh = False
        self.graph.replay()
        for host, (flag, _) in zip(self._host_flags, self._flags):
            host.copy_(flag, non_blocking=True)
        if self._flags:
            self._flag_event = torch.cuda.Event()
            self._flag_event.record()
        return self.loss

    def flush(self):
        """Raises for an out-of-range token id seen by the last replay."""
        self._check_previous()
