"""The acting step of a sequence model as a HIP graph.

Acting calls the model once per environment step with T = 1 (ppo.py:105-143): a torso of a few blocks is
then some hundred launches of kernels that run a few microseconds each, and the step takes as long as
the host needs to issue them (2.3 ms for configuration 5's torso at 1024 environments, of which the
device is busy for 0.6).  ``GraphedStep`` records one step -- (inputs (B,1,F), done (B,1), carry) ->
(next carry, y), without gradients -- into a graph over fixed buffers and replays it: the same kernels,
the same results bit for bit, one launch.

    act = GraphedStep(torso, batch=1024, features=256, autocast=torch.bfloat16)
    for obs, done in rollout:               # obs (B,1,F), done (B,1)
        y = act(obs, done)                  # valid until the next call
    carry = act.carry                       # the model's carry pytree (copies)

Everything the step does must be capturable: no host synchronisation, no data-dependent shapes.  The
modules of ``sequence_models`` are; the library's kernels take the capturing stream like any other.

Under autocast every dense layer casts its weight on every call -- in a step of 0.7 ms that is a seventh
of the device's time, for weights that change once per update.  The graph therefore runs on copies of the
matrices in the autocast dtype, which a call refreshes only for parameters that have been written since
(``torch.Tensor._version``, which optimisers and ``load_state_dict`` advance; ``sync_weights()`` after
anything that writes through ``.data``).
"""
from __future__ import annotations

import contextlib

import torch

from .functional import step_in_place


def _leaves(tree, out):
    if isinstance(tree, (tuple, list)):
        for v in tree:
            _leaves(v, out)
    elif isinstance(tree, dict):
        for k in sorted(tree):
            _leaves(tree[k], out)
    elif tree is not None:
        out.append(tree)
    return out


def _map(fn, tree):
    if isinstance(tree, (tuple, list)):
        items = [_map(fn, v) for v in tree]
        return type(tree)(*items) if hasattr(tree, "_fields") else type(tree)(items)   # named tuples keep their type
    if isinstance(tree, dict):
        return {k: _map(fn, v) for k, v in tree.items()}
    return None if tree is None else fn(tree)


class GraphedStep:
    """One no-gradient step of ``model`` at a fixed batch size, captured once and replayed.

    model: a SequenceModel (``(inputs, done, initial_carry) -> (next_carry, y)``, ``initialize_carry``).
    autocast: dtype of a ``torch.autocast`` region around the step, or None.
    The carry lives in buffers of this object: ``reset()`` puts the model's initial carry there, ``set_carry``
    a given one; the matrix states are updated in them by the step kernels, every other leaf of the step's next
    carry is copied over them after the call.
    """

    def __init__(self, model, batch, features, autocast=None, device="cuda", warmup=3):
        self.model, self.autocast = model, autocast
        # matrices in the dtype the products run in; vectors (norm scales, biases) stay as they are
        self._shadow, self._seen = {}, {}
        if autocast is not None:
            for name, p in model.named_parameters():
                if p.dim() >= 2 and p.is_floating_point():
                    self._shadow[name] = p.detach().to(autocast)
                    self._seen[name] = p._version
        self._params = dict(model.named_parameters())
        self._x = torch.zeros(batch, 1, features, device=device)
        self._done = torch.zeros(batch, 1, dtype=torch.bool, device=device)
        with torch.no_grad():
            self._carry = _map(lambda t: t.detach().clone(), model.initialize_carry(None, (batch, features)))
        self._initial = _map(lambda t: t.clone(), self._carry)
        # the kernels' per-device set-up and the array library's lazy initialisations happen on a side stream first:
        # nothing of that kind may fall into the capture
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):
            for _ in range(warmup):
                self._run()
        torch.cuda.current_stream(device).wait_stream(side)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._next, self._y = self._run()
        held, made = _leaves(self._carry, []), _leaves(self._next, [])
        if len(held) != len(made) or any(a.shape != b.shape for a, b in zip(held, made)):
            raise ValueError("the step's next carry does not have the leaves of the carry it was given")
        if not all(t.is_cuda for t in held):
            raise ValueError("the model's carry must live on the device")
        # leaves the step has updated in place need no copy back
        same = lambda a, b: a.data_ptr() == b.data_ptr() and a.stride() == b.stride() and a.dtype == b.dtype   # noqa: E731
        self._pairs = [(a, b) for a, b in zip(held, made) if not same(a, b)]
        self.reset()

    def _run(self):
        ctx = torch.autocast("cuda", dtype=self.autocast) if self.autocast is not None else contextlib.nullcontext()
        # the carry's buffers are this object's own: the single-step kernels update the states where they lie
        with torch.no_grad(), ctx, step_in_place():
            if self._shadow:
                return torch.func.functional_call(self.model, self._shadow, (self._x, self._done, self._carry))
            return self.model(self._x, self._done, self._carry)

    def sync_weights(self, force=True):
        """Refresh the graph's copies of the weight matrices: all of them, or (force=False) those written since
        the last refresh."""
        with torch.no_grad():
            for name, copy in self._shadow.items():
                p = self._params[name]
                if force or p._version != self._seen[name]:
                    copy.copy_(p)
                    self._seen[name] = p._version

    def __call__(self, inputs, done):
        """inputs (B,1,F), done (B,1) bool or float -> y (B,1,...), a buffer of this object that the next call
        overwrites."""
        self.sync_weights(force=False)
        self._x.copy_(inputs)
        self._done.copy_(done != 0 if done.dtype != torch.bool else done)
        self._graph.replay()
        for dst, src in self._pairs:
            dst.copy_(src)
        return self._y

    @property
    def carry(self):
        """The carry after the last call, as copies in the model's pytree."""
        return _map(lambda t: t.clone(), self._carry)

    def set_carry(self, carry):
        held, given = _leaves(self._carry, []), _leaves(carry, [])
        if len(held) != len(given):
            raise ValueError(f"a carry of {len(given)} leaves for a model whose carry has {len(held)}")
        for dst, src in zip(held, given):
            dst.copy_(src)

    def reset(self):
        self.set_carry(self._initial)
