"""`@flex_rnn.jit`: the user-facing decorator.

Same surface and semantics as the reference class
(/root/reference/flex_rnn/jit.py:7-84): attributes `step, ninputs, nstates,
noutputs, apply, forward_func, backward_func, fw_meta, bw_meta`, methods
`naive(*args, dtype=)`, `naive_fp64(*args)`, and `obj(*inputs, *states) ->
(*outputs, *final_states)`.  Two dispatcher ops are registered per instance,
`flex_rnn::fw_<id>` and `flex_rnn::bw_<id>`, with fake (meta) implementations and an
autograd formula, so the object composes with `torch.compile` without graph
breaks.  Kernels are built lazily on the first real call; a later call with other
shapes, strides or dtypes fails the metadata check, as in the reference.

Beyond the reference: `jit(step, dynamic=True)` (or `jit.dynamic(step)`) keeps one plan per
distinct (shape, stride, dtype) signature of the arguments instead of failing.  The kernels
take B, T, H, M and all strides at run time, so signatures that lead to the same tile reuse
the same cached code objects and only pay for tracing and planning.
"""
from __future__ import annotations

import inspect
import uuid
import weakref

import torch as th

from .planner import build_twopass, split_list, verify_meta


def _tup(x):
    return x if type(x) == tuple else (x,)


def _sig(tensors):
    return tuple((tuple(int(n) for n in t.shape), tuple(int(n) for n in t.stride()), t.dtype) for t in tensors)


class jit:
    _instances = weakref.WeakValueDictionary()      # dispatcher name of the forward operator -> its jit object

    @classmethod
    def instance_of(cls, op_name: str):
        """The jit object whose forward operator has this dispatcher name (`flex_rnn::fw_<id>`, with or without an
        overload suffix), or None: lets a traced graph be mapped back to the objects it calls."""
        return cls._instances.get(op_name.split('.')[0])

    def __init__(self, step, n_step_args=None, dynamic=False):
        self.step = step
        self.forward_func = self.backward_func = None
        self.is_dynamic = bool(dynamic)
        self._entries = {}        # dynamic mode: argument signature -> plan entry
        self._by_id = {}          # dynamic mode: entry number -> plan entry (see `_tag`)
        if n_step_args is None:
            n_step_args = len(inspect.signature(step).parameters)
        # arity: run the step once on 1x1 meta tensors (jit.py:13-16)
        y, s = step(*[th.empty(1, 1, device='meta') for _ in range(n_step_args)])
        self.noutputs, self.nstates = len(y), len(s)
        self.ninputs = n_step_args - self.nstates
        self.apply = self.build_call()

    def __call__(self, *args):
        return self.apply(*args)

    @classmethod
    def dynamic(cls, step, n_step_args=None):
        """Decorator form of `jit(step, dynamic=True)`."""
        return cls(step, n_step_args, dynamic=True)

    def _entry(self, inputs, state, dry):
        """Dynamic mode: the plan entry for this argument signature, planned (`dry`) or built."""
        key = _sig(inputs) + _sig(state)
        e = self._entries.setdefault(key, {})
        if dry:
            if 'fw_meta' not in e:
                e['fw_meta'], e['bw_meta'] = build_twopass(self.step, inputs, state, dryrun=True)
        elif 'forward' not in e:
            e['forward'], e['backward'], e['fw_meta'], e['bw_meta'] = build_twopass(self.step, inputs, state)
        if 'id' not in e:
            e['id'] = len(self._by_id) + 1
            self._by_id[e['id']] = e
        self.fw_meta, self.bw_meta = e['fw_meta'], e['bw_meta']
        self.forward_func, self.backward_func = e.get('forward'), e.get('backward')
        return e

    @staticmethod
    def _tag(e, device):
        """Dynamic mode: a hidden result without elements whose *shape* `[0, entry number]` names the plan
        entry of a forward call.  It is saved for backward with the checkpoints, so the backward operator
        finds the plan of exactly that forward call from static metadata alone (it also survives
        tracing by `torch.compile`): two signatures that differ only in the state's dtype or strides
        have the same inputs and checkpoint shapes and could not be told apart by those."""
        return th.empty((0, e['id']), dtype=th.uint8, device=device)

    def _bw_entry(self, tag):
        assert tag.ndim == 2 and tag.shape[0] == 0 and tag.shape[1] in self._by_id, \
            'backward called with tensors no forward call has produced'
        return self._by_id[tag.shape[1]]

    def infer(self, *args):
        """Outputs and final states without the ability to differentiate: the forward kernel then
        writes neither state checkpoints nor the per-step row sums the backward pass would need
        (an addition to the reference's interface, for inference and decoding loops).  Same
        arguments and results as a call; not recorded by autograd."""
        inputs, state = split_list(args, [self.ninputs, self.nstates])
        with th.no_grad():
            if self.is_dynamic:
                fwd = self._entry(inputs, state, dry=False)['forward']
            else:
                if self.forward_func is None:
                    self.forward_func, self.backward_func, self.fw_meta, self.bw_meta = \
                        build_twopass(self.step, inputs, state)
                fwd = self.forward_func
            return fwd.forward_only(inputs, state)

    def segmented(self, *args, segment: int):
        """The results (and gradients) of a call, computed `segment` timesteps at a time under activation
        checkpointing (an addition to the reference's interface, for sequences whose hidden buffers do not fit):
        only the states at the segment boundaries are kept for the backward pass, which runs a segment's forward
        kernel again just before that segment's backward kernels.  The hidden buffers - fp32 state and d-state
        checkpoints every 16 timesteps, saved row sums - then exist for one segment at a time instead of the whole
        sequence, at the price of one more forward pass.  Segments are planned like calls of a `dynamic` instance."""
        from torch.utils.checkpoint import checkpoint
        inputs, state = split_list(args, [self.ninputs, self.nstates])
        assert segment >= 1
        T = max(i.shape[1] for i in inputs)
        if getattr(self, '_segments', None) is None:
            self._segments = self if self.is_dynamic else jit(self.step, self.ninputs + self.nstates, dynamic=True)
        outs = [[] for _ in range(self.noutputs)]
        for t0 in range(0, T, segment):
            part = [x[:, t0:t0 + segment] if x.shape[1] != 1 else x for x in inputs]
            if isinstance(self._segments, jit) and part[0].is_cuda and not isinstance(part[0], th._subclasses.FakeTensor):
                # (plans are traced with torch.func, which refuses to run under the saved-tensor hooks of `checkpoint`)
                self._segments._entry(part, list(state), dry=False)
            res = checkpoint(self._segments.apply, *part, *state, use_reentrant=False)
            for k in range(self.noutputs):
                outs[k].append(res[k])
            state = tuple(res[self.noutputs:])
        if T == 0:
            return self._segments.apply(*args)
        return (*[th.cat(o, dim=1) for o in outs], *state)

    # ------------------------------------------------------------------ plain per-timestep loop
    def naive(self, *args, dtype=th.float32):
        """Pure-PyTorch per-timestep loop with the compiled path's calling convention
        (jit.py:23-36): inputs are cast to `dtype`, the initial state is not; outputs
        come back in the step's output dtype under `dtype` inputs, final states in the
        layout of the initial states."""
        inputs, state0 = split_list(args, [self.ninputs, self.nstates])
        state = state0
        T = max(i.shape[1] for i in inputs)
        output = None
        for t in range(T):
            inputs_t = tuple(i.expand(-1, T, -1, -1, -1)[:, t].to(dtype) for i in inputs)
            output_t, state = self.step(*inputs_t, *state)
            output_t, state = _tup(output_t), _tup(state)
            if output is None:
                output = tuple(th.empty(o.shape[0], T, o.shape[1], o.shape[2], dtype=o.dtype, device=o.device)
                               for o in output_t)
            for dst, src in zip(output, output_t):
                dst[:, t] = src.squeeze(-1)
        state = tuple(th.empty_like(x).copy_(y) for x, y in zip(state0, state))
        return (*output, *state)

    def naive_fp64(self, *args):
        return self.naive(*args, dtype=th.double)

    # --------------------------------------------------------------- dispatcher
    def build_call(self):
        uid = uuid.uuid4().hex
        nin, nst, nout = self.ninputs, self.nstates, self.noutputs
        naux = 1        # all saved row-sums travel in one packed tensor (jit.py:43)
        ntag = 1 if self.is_dynamic else 0      # dynamic mode: one more hidden result, see `_tag`

        def metas(meta, device):
            return tuple(th.empty_strided(shape, stride, dtype=dtype, device=device) for shape, stride, dtype in meta)

        checked = {}        # id(meta) -> (meta, its meta tensors): what results are compared with on every call

        def expected(meta):
            hit = checked.get(id(meta))
            if hit is None or hit[0] is not meta:
                hit = checked[id(meta)] = (meta, metas(meta, 'meta'))
            return hit[1]

        fw_schema = '(' + ', '.join(f'Tensor x{i}' for i in range(nin + nst)) + ') -> (' \
            + ', '.join(['Tensor'] * (nout + 2 * nst + naux + ntag)) + ')'

        @th.library.custom_op('flex_rnn::fw_' + uid, mutates_args=(), schema=fw_schema)
        def apply(*args):
            inputs, state = split_list(args, [nin, nst])
            if self.is_dynamic:
                e = self._entry(inputs, state, dry=False)
                r = e['forward'](inputs, state)
                verify_meta(r, expected(e['fw_meta']))
                return (*r, self._tag(e, args[0].device))
            if self.forward_func is None:
                self.forward_func, self.backward_func, self.fw_meta, self.bw_meta = \
                    build_twopass(self.step, inputs, state)
            r = self.forward_func(inputs, state)
            verify_meta(r, expected(self.fw_meta))
            return r

        @apply.register_fake
        def _(*args):
            inputs, state = split_list(args, [nin, nst])
            if self.is_dynamic:
                e = self._entry(inputs, state, dry=True)
                return (*metas(e['fw_meta'], args[0].device), self._tag(e, args[0].device))
            if not hasattr(self, 'fw_meta'):
                self.fw_meta, self.bw_meta = build_twopass(self.step, inputs, state, dryrun=True)
            return metas(self.fw_meta, args[0].device)

        bw_schema = '(' + ', '.join(f'Tensor x{i}' for i in range(nout + 2 * nst + nin + naux + ntag)) + ') -> (' \
            + ', '.join(['Tensor'] * (nin + nst)) + ')'

        @th.library.custom_op('flex_rnn::bw_' + uid, mutates_args=(), schema=bw_schema)
        def backward_inner(*args):
            doutput, dstateT, inputs, state_store, aux, tag = split_list(args, [nout, nst, nin, nst, naux, ntag])
            if self.is_dynamic:
                e = self._bw_entry(tag[0])
                dinputs, dstate0 = e['backward'](doutput, dstateT, inputs, state_store, aux)
                verify_meta(dinputs + dstate0, expected(e['bw_meta']))
                return (*dinputs, *dstate0)
            dinputs, dstate0 = self.backward_func(doutput, dstateT, inputs, state_store, aux)
            verify_meta(dinputs + dstate0, expected(self.bw_meta))
            return (*dinputs, *dstate0)

        @backward_inner.register_fake
        def _(*args):
            if self.is_dynamic:
                return metas(self._bw_entry(args[-1])['bw_meta'], args[0].device)
            return metas(self.bw_meta, args[0].device)

        def setup_context(ctx, inputs, output):
            ctx.set_materialize_grads(False)
            ctx.save_for_backward(*inputs[:nin], *output[nout + nst:])
            ctx.output_meta = tuple((o.shape, o.stride(), o.dtype) for o in output[:nout + nst])

        def backward(ctx, *grads):
            grads = list(grads)
            for i, (shape, stride, dtype) in enumerate(ctx.output_meta):
                if grads[i] is None:
                    grads[i] = th.empty_strided(shape, stride, dtype=dtype, device=ctx.saved_tensors[0].device).zero_()
            return backward_inner(*grads[:nout + nst], *ctx.saved_tensors)

        apply.register_autograd(backward, setup_context=setup_context)
        self._fw_op, self._bw_op = apply, backward_inner
        jit._instances['flex_rnn::fw_' + uid] = self
        return lambda *args: apply(*args)[:nout + nst]


def simplified_naive(step, *args):
    """Single-state, single-output loop shown in the reference's README (jit.py:86-94)."""
    inputs, state = args[:-1], args[-1]
    T = max(i.shape[1] for i in inputs)
    ys = []
    for t in range(T):
        xs = [i.expand(-1, T, -1, -1, -1)[:, t].float() for i in inputs]
        y, state = step(*xs, state)
        ys.append(y)
    return th.stack(ys, dim=1).squeeze(-1), state
