"""Decorator surface, operand validation, dry-run metadata and fake-tensor behaviour - the
parts of the boundary that need no GPU."""
import pytest
import torch as th

import flex_rnn_amd
from flex_rnn_amd import ops, planner
from flex_rnn_amd.planner import split_list, verify_meta

import cases


def test_arity_inference_and_surface():
    f = flex_rnn_amd.jit(ops.rwkv7)
    assert (f.ninputs, f.nstates, f.noutputs) == (6, 1, 1)
    g = flex_rnn_amd.jit(ops.rwkv4)
    assert (g.ninputs, g.nstates, g.noutputs) == (4, 3, 1)
    h = flex_rnn_amd.jit(ops.mlstm_gates)
    assert (h.ninputs, h.nstates, h.noutputs) == (2, 1, 3)
    for attr in ('step', 'apply', 'forward_func', 'backward_func', 'naive', 'naive_fp64', 'build_call'):
        assert hasattr(f, attr)
    assert f.forward_func is None and f.backward_func is None        # nothing compiled yet
    assert flex_rnn_amd.__version__ == '0.2'
    assert callable(flex_rnn_amd.check_grad) and callable(flex_rnn_amd.benchmark)
    # explicit arity for a step with *args
    k = flex_rnn_amd.jit(lambda *a: ops.gla(*a), n_step_args=5)
    assert (k.ninputs, k.nstates) == (4, 1)


def test_apply_is_reassignable():
    f = flex_rnn_amd.jit(ops.gla)
    step, xs, ss = cases.make_inputs('gla', 1, 4, 1, 4, 4, dtype=th.float32)
    f.apply = f.naive_fp64
    y, S = f(*xs, *ss)
    assert y.dtype == th.float64 and y.shape == (1, 4, 1, 4)


def test_split_list_and_verify_meta():
    assert split_list([1, 2, 3, 4], [1, 3]) == [[1], [2, 3, 4]]
    with pytest.raises(AssertionError):
        split_list([1, 2, 3], [1, 1])
    a = th.empty(2, 1, 4)
    verify_meta([a], [th.empty(2, 1, 4).as_strided((2, 1, 4), (4, 99, 1))])     # stride of a size-1 dim is ignored
    with pytest.raises(AssertionError, match='shape'):
        verify_meta([a], [th.empty(2, 2, 4)])
    with pytest.raises(AssertionError, match='stride'):
        verify_meta([a], [th.empty(4, 1, 2).permute(2, 1, 0)])
    with pytest.raises(AssertionError, match='dtype'):
        verify_meta([a], [th.empty(2, 1, 4, dtype=th.bfloat16)])


def test_operand_validation_messages():
    S = th.zeros(2, 3, 4, 8)
    q = th.zeros(2, 5, 3, 1, 8)
    with pytest.raises(AssertionError, match='invalid shape'):
        planner.classify([th.zeros(2, 5, 3, 8)], [S])
    with pytest.raises(AssertionError, match='incompatible'):
        planner.classify([q, th.zeros(2, 5, 2, 4, 1)], [S])
    with pytest.raises(AssertionError, match='both a matrix'):
        planner.classify([q, th.zeros(2, 5, 3, 4, 8)], [S])
    with pytest.raises(AssertionError, match='!='):
        planner.classify([q], [th.zeros(2, 1, 4, 8)])
    with pytest.raises(AssertionError, match='dtype'):
        planner.classify([q.to(th.int32)], [S])
    dims, cls, bc = planner.classify([q, th.zeros(2, 5, 3, 4, 1), th.zeros(1, 1, 3, 1, 1), th.zeros(1, 1, 3, 4, 8)], [S])
    assert dims == [2, 5, 3, 4, 8] and cls == ['row', 'col', 'scalar', 'mat']
    assert bc == [(False, False, False), (False, False, False), (True, True, False), (True, True, False)]


def test_dryrun_metadata():
    step, xs, ss = cases.make_inputs('rwkv7', 2, 32, 3, 16, 32, dtype=th.bfloat16)
    ss = [s.float().mT.contiguous().mT for s in ss]                 # transposed-stride state
    fw_meta, bw_meta = planner.build_twopass(step, xs, ss, dryrun=True)
    (ysh, yst, ydt), (ssh, sst, sdt), (cksh, _, ckdt), (ash, _, adt) = fw_meta
    assert tuple(ysh) == (2, 32, 3, 16) and ydt == th.bfloat16           # step ends in .to(r.dtype)
    assert tuple(ssh) == (2, 3, 16, 32) and tuple(sst) == tuple(ss[0].stride()) and sdt == th.float32
    assert tuple(cksh) == (2, 3, 2, 16, 32) and ckdt == th.float32       # a checkpoint every 16 steps
    assert tuple(ash) == (1, 2, 3, 32, 16) and adt == th.float32         # one saved row sum per step
    assert len(bw_meta) == 7
    for (sh, st, dt), x in zip(bw_meta, xs + ss):
        assert tuple(sh) == tuple(x.shape) and dt == x.dtype


def test_fake_tensor_mode_uses_dry_run():
    from torch._subclasses.fake_tensor import FakeTensorMode
    f = flex_rnn_amd.jit(ops.delta_rule)
    step, xs, ss = cases.make_inputs('delta_rule', 2, 16, 2, 8, 8, dtype=th.float32)
    with FakeTensorMode() as mode:
        fx = [mode.from_tensor(x) for x in xs]
        fs = [mode.from_tensor(s) for s in ss]
        y, S = f(*fx, *fs)
    assert tuple(y.shape) == (2, 16, 2, 8) and tuple(S.shape) == (2, 2, 8, 8)
    assert f.forward_func is None            # nothing was compiled or launched
    assert hasattr(f, 'fw_meta') and hasattr(f, 'bw_meta')


def test_dynamic_mode_plans_one_entry_per_signature():
    from torch._subclasses.fake_tensor import FakeTensorMode
    f = flex_rnn_amd.jit.dynamic(ops.delta_rule)
    assert f.is_dynamic and not flex_rnn_amd.jit(ops.delta_rule).is_dynamic
    shapes = []
    for dims in ((2, 16, 2, 8, 8), (1, 40, 2, 8, 8), (2, 16, 2, 8, 8)):
        step, xs, ss = cases.make_inputs('delta_rule', *dims, dtype=th.float32)
        with FakeTensorMode() as mode:
            y, S = f(*[mode.from_tensor(x) for x in xs], *[mode.from_tensor(s) for s in ss])
        shapes.append((tuple(y.shape), tuple(S.shape)))
    assert shapes[0] == ((2, 16, 2, 8), (2, 2, 8, 8)) and shapes[1] == ((1, 40, 2, 8), (1, 2, 8, 8))
    assert len(f._entries) == 2 and f.forward_func is None
    # a strict instance keeps the first signature's metadata
    g = flex_rnn_amd.jit(ops.delta_rule)
    for dims in ((2, 16, 2, 8, 8), (1, 40, 2, 8, 8)):
        step, xs, ss = cases.make_inputs('delta_rule', *dims, dtype=th.float32)
        with FakeTensorMode() as mode:
            y, S = g(*[mode.from_tensor(x) for x in xs], *[mode.from_tensor(s) for s in ss])
    assert tuple(y.shape) == (2, 16, 2, 8)


def test_dynamic_mode_backward_finds_the_plan_of_its_own_forward_call():
    """Two signatures that differ only in the state's dtype (or only in its strides) have the same inputs
    and checkpoint shapes.  The backward operator must still run the plan of the forward call it belongs to:
    the hidden tag result carries the entry number in its shape."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    f = flex_rnn_amd.jit.dynamic(ops.delta_rule)
    step, xs, ss = cases.make_inputs('delta_rule', 2, 16, 2, 8, 8, dtype=th.float32)
    variants = [ss[0], ss[0].to(th.bfloat16), ss[0].transpose(-1, -2).contiguous().transpose(-1, -2)]
    with FakeTensorMode() as mode:
        fx = [mode.from_tensor(x) for x in xs]
        outs = []
        for s0 in variants:
            fs = mode.from_tensor(s0).requires_grad_()
            outs.append((fs, f(*fx, fs)))
        assert len(f._entries) == 3 and sorted(f._by_id) == [1, 2, 3]
        # backward of the calls in an order other than the forward calls'
        for k in (0, 2, 1):
            fs, (y, S) = outs[k]
            (g,) = th.autograd.grad([y, S], [fs], [th.ones_like(y), th.ones_like(S)])
            assert g.dtype == variants[k].dtype and g.stride() == variants[k].stride(), k
    with pytest.raises(AssertionError, match='no forward call has produced'):
        f._bw_entry(th.empty(0, 7, dtype=th.uint8))


def test_infer_is_part_of_the_surface_and_has_no_cpu_fallback(runtime_lib):
    if th.cuda.is_available():
        pytest.skip('a GPU is present')
    f = flex_rnn_amd.jit(ops.delta_rule)
    step, xs, ss = cases.make_inputs('delta_rule', 2, 16, 2, 8, 8, dtype=th.float32)
    with pytest.raises(Exception) as e:
        f.infer(*xs, *ss)
    assert 'GPU' in str(e.value) or 'HIP' in str(e.value) or 'hip' in str(e.value)


def test_compiled_path_has_no_cpu_fallback(runtime_lib):
    if th.cuda.is_available():
        pytest.skip('a GPU is present')
    f = flex_rnn_amd.jit(ops.delta_rule)
    step, xs, ss = cases.make_inputs('delta_rule', 1, 16, 1, 16, 16, dtype=th.float32)
    with pytest.raises((RuntimeError, AssertionError)):
        f(*xs, *ss)


def test_unsupported_op_is_named():
    def bad(x, S):
        S = S + th.cumsum(x, -1)
        return S.sum(-1, True), S
    with pytest.raises(NotImplementedError, match='cumsum'):
        planner.make_plan(bad, [th.zeros(1, 2, 1, 1, 4)], [th.zeros(1, 1, 4, 4)])


def test_drop_in_alias_package():
    import flex_rnn
    assert flex_rnn.jit is flex_rnn_amd.jit and flex_rnn.check_grad is flex_rnn_amd.check_grad


def test_dynamo_traces_through_the_op_without_graph_break(runtime_lib):
    """torch.compile sees one opaque op: the captured graph holds a single flex_rnn::fw_* call
    and no graph break occurs.  (Running it needs a GPU; only the capture is checked here.)"""
    if th.cuda.is_available():
        pytest.skip('covered by the GPU test')
    f = flex_rnn_amd.jit(ops.delta_rule)
    step, xs, ss = cases.make_inputs('delta_rule', 1, 16, 2, 8, 8, dtype=th.float32)
    graphs = []

    def backend(gm, example_inputs):
        graphs.append(gm)
        return gm.forward

    def layer(q, k, v, beta, S):
        y, S = f(q * 2, k, v, beta, S)
        return y + 1, S

    compiled = th.compile(layer, backend=backend, fullgraph=True)
    with pytest.raises((RuntimeError, AssertionError)):      # no GPU: the real kernel cannot run
        compiled(*xs, *ss)
    assert len(graphs) == 1
    targets = [str(n.target) for n in graphs[0].graph.nodes if n.op == 'call_function']
    assert sum('flex_rnn.fw_' in t for t in targets) == 1, targets


def test_fixed_pick_switch_is_parsed(monkeypatch):
    from flex_rnn_amd import launch
    monkeypatch.delenv('FLEX_RNN_PICK', raising=False)
    assert launch._fixed_picks() == {}
    monkeypatch.setenv('FLEX_RNN_PICK', 'frnn_fw=3, frnn_bw1=1')
    assert launch._fixed_picks() == {'frnn_fw': 3, 'frnn_bw1': 1}


def test_row_kernel_candidate_tiles_are_valid():
    """Every candidate tile of the row kernels covers the state row, keeps the workgroup within the
    state's rows and passes the planner's own check; the headline shape offers the wide-column tile."""
    import dataclasses
    from flex_rnn_amd import launch, planner, prebuild
    for name in ('rwkv7', 'mamba2', 'gated_delta_rule', 'mamba1'):
        plan = prebuild.plan_for(name)
        for reverse in (False, True):
            tiles = launch.row_kernel_tiles(plan, reverse)
            assert tiles[0][:2] == (plan.tile.L, plan.tile.C) and len(set(tiles)) == len(tiles) <= 5
            for L, C, r, w in tiles:
                assert L * C == plan.NP and (64 // L) * r * w <= max(plan.M, (64 // L) * r)
                t = dataclasses.replace(plan.tile, L=L, C=C)
                t = dataclasses.replace(t, R1=r, W1=w) if reverse else dataclasses.replace(t, R=r, W=w)
                planner.check_tile(t, plan.H, plan.NP, plan.part)
            variants = launch.row_kernel_variants(plan, reverse)
            assert len(variants) >= len(tiles) and len({repr(v) for v in variants}) == len(variants)
            assert variants[0] == dataclasses.replace(variants[0], NB=plan.tile.NB, UR=plan.tile.UR)     # first: the plan's own tile
            for v in variants:
                planner.check_tile(v, plan.H, plan.NP, plan.part)
    assert (8, 16, 2, 8) in launch.row_kernel_tiles(prebuild.plan_for('rwkv7'), False)
    # large problems also time the first tile with a register budget of half a SIMD's file; knob values out of range are refused
    plan = prebuild.plan_for('rwkv7')
    assert any(v.WN == 2 for v in launch.row_kernel_variants(plan, False)) and all(v.WN == 0 for v in launch.row_kernel_variants(
        prebuild.plan_for('rwkv7', (2, 64, 2, 128, 128)), False))
    for bad in (dict(WN=9), dict(DF=2), dict(NB=4), dict(UR=0)):
        with pytest.raises(AssertionError):
            planner.check_tile(dataclasses.replace(plan.tile, **bad), plan.H, plan.NP, plan.part)


def test_tile_heuristic_gives_valid_tiles_for_ragged_shapes():
    """Row counts and widths that are not powers of two, single rows, narrow and wide states: the heuristic's tile
    passes the planner's own check (a row count of 24 once gave three waves per workgroup)."""
    from flex_rnn_amd import prebuild
    for name in ('mamba1', 'mamba2', 'rwkv7', 'gated_delta_rule', 'delta_rule'):
        for M in (1, 3, 24, 40, 100, 192):
            for N in ((8, 16) if name == 'mamba1' else (16, 48, 128)):
                for B, T, H in ((1, 19, 1), (8, 1024, 32)):
                    plan = prebuild.plan_for(name, (B, T, H, M, N))
                    planner.check_tile(plan.tile, plan.H, plan.NP, plan.part)


def test_timed_picks_are_kept_beside_the_cache(tmp_path, monkeypatch):
    """The choice among candidate builds is stored per (kernel, candidates, device, B, H, M) - not per
    sequence length - and found again by a fresh process (here: a fresh `_Picks`)."""
    from flex_rnn_amd import launch, prebuild
    from flex_rnn_amd.emit_hip import KernelSpec
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    builds = [(KernelSpec('frnn_fw', f'// candidate {i}', [], 64, ('1', '1', '1')), None, None) for i in range(3)]
    long_plan = prebuild.plan_for('rwkv7', (2, 64, 2, 128, 128))
    short_plan = prebuild.plan_for('rwkv7', (2, 32, 2, 128, 128))
    other_plan = prebuild.plan_for('rwkv7', (4, 64, 2, 128, 128))
    key = launch.PICKS.key('frnn_fw', builds, 'dev', long_plan)
    assert key == launch.PICKS.key('frnn_fw', builds, 'dev', short_plan)
    assert key != launch.PICKS.key('frnn_fw', builds, 'dev', other_plan)
    assert key != launch.PICKS.key('frnn_fw', builds[:2], 'dev', long_plan)
    assert key != launch.PICKS.key('frnn_fw', builds, 'other dev', long_plan)
    a = launch._Picks()
    assert a.get(key, 3) is None
    a.put(key, 2, [0.5, float('inf'), 0.25])
    assert a.get(key, 3)['index'] == 2
    b = launch._Picks()                       # another process
    rec = b.get(key, 3)
    assert rec['index'] == 2 and rec['ms'] == [0.5, None, 0.25]
    assert b.get(key, 2) is None              # a stored index that the candidate list no longer has is ignored
    b.put('other', 0, [1.0])
    assert launch._Picks().get(key, 3)['index'] == 2 and launch._Picks().get('other', 1)['index'] == 0


def test_compiled_plan_keeps_its_host_interface():
    """The host object behind `forward` / `backward` (the CPU harness swaps only its two device-facing methods)."""
    from flex_rnn_amd.launch import CompiledPlan
    for m in ('_launch', '_tune', '_select', '_register', '_install', '_row_builds', 'forward', 'forward_only', 'backward',
              'static_layout', 'launch_static'):
        assert callable(getattr(CompiledPlan, m, None)), m


def test_segmented_call_slices_time_and_carries_the_state():
    """`jit.segmented` (the compiled operator replaced by the plain loop here, which takes the same arguments): outputs,
    final states and all gradients equal those of one call over the whole sequence; time-independent inputs are not
    sliced; the last segment may be shorter."""
    step, xs, ss = cases.make_inputs('mamba', 2, 11, 2, 4, 4, dtype=th.float64)
    f = flex_rnn_amd.jit(step)
    f._segments = type('Loop', (), {'apply': staticmethod(lambda *a: f.naive(*a, dtype=th.float64))})()
    xg = [x.clone().requires_grad_() for x in xs]
    sg = [s.clone().requires_grad_() for s in ss]
    whole = f.naive(*xg, *sg, dtype=th.float64)
    gy = [th.randn_like(r) for r in whole]
    want = th.autograd.grad(whole, xg + sg, gy)
    for segment in (4, 11, 16, 1):
        got = f.segmented(*xg, *sg, segment=segment)
        assert all(a.shape == b.shape for a, b in zip(got, whole))
        assert all(th.allclose(a, b, rtol=0, atol=1e-12) for a, b in zip(got, whole)), segment
        grads = th.autograd.grad(got, xg + sg, gy)
        assert all(th.allclose(a, b, rtol=0, atol=1e-10) for a, b in zip(grads, want)), segment


def test_shipped_picks_are_well_formed_and_name_existing_candidates():
    """The timed choices shipped for the benchmark workloads: one record per key with an index into the candidate list
    and one timing per candidate; those whose key matches the current row-kernel sources index an existing candidate
    (a key for other sources is ignored at run time and the kernel is timed again)."""
    import json
    from flex_rnn_amd import launch, prebuild
    shipped = json.load(open(launch.PICKS.SHIPPED))
    assert shipped and all(isinstance(v['index'], int) and 0 <= v['index'] < max(len(v['ms']), 1) for v in shipped.values())
    devices = {k.split('|')[2] for k in shipped}
    matched = 0
    for dev in devices:
        for wl in ('rwkv7', 'mamba1'):
            plan = prebuild.plan_for(wl)
            for kname, specs in (('frnn_fw', launch.row_kernel_specs(plan, False)), ('frnn_bw1', launch.row_kernel_specs(plan, True))):
                key = launch.PICKS.key(kname, [(s, None, None) for s in specs], dev, plan)
                if key in shipped:
                    matched += 1
                    assert shipped[key]['index'] < len(specs) == len(shipped[key]['ms'])
    # a cache directory without choices of its own starts from the shipped ones
    import os, tempfile
    old = os.environ.get('FLEX_RNN_CACHE')
    with tempfile.TemporaryDirectory() as tmp:
        os.environ['FLEX_RNN_CACHE'] = tmp
        try:
            key = next(iter(shipped))
            assert launch._Picks().get(key, len(shipped[key]['ms']))['index'] == shipped[key]['index']
        finally:
            os.environ.pop('FLEX_RNN_CACHE') if old is None else os.environ.__setitem__('FLEX_RNN_CACHE', old)
    if not matched:
        pytest.skip('the shipped choices were timed on other kernel sources; they are ignored until exported again')


def test_kept_row_sums_and_deeper_staging_are_candidates_where_they_apply():
    """`TileConfig.KS` is a timed candidate of large problems only, per kernel (bit 0 forward, bit 1 reverse scan), and the
    emitter ignores it where a group of lanes is too small to keep a block's steps; a candidate tile with more waves than the
    plan's own stages as many timesteps as its larger LDS share holds."""
    import dataclasses
    import torch as th
    import flex_rnn_amd
    from flex_rnn_amd import examples, launch, planner, prebuild
    from flex_rnn_amd.emit_hip import Emitter
    plan = prebuild.plan_for('rwkv7')
    for reverse in (False, True):
        bit = 2 if reverse else 1
        variants = launch.row_kernel_variants(plan, reverse)
        assert any(v.KS & bit for v in variants) and not any(v.KS & (3 ^ bit) for v in variants)
    assert all(v.KS == 0 for v in launch.row_kernel_variants(prebuild.plan_for('rwkv7', (2, 64, 2, 128, 128)), False))
    kept = Emitter(dataclasses.replace(plan, tile=dataclasses.replace(plan.tile, KS=3)))
    assert 'k_y0' in kept.fw().source and 'k_y0' in kept.fw(save=False).source and 'k_da0' in kept.bw1().source
    assert 'k_y0' not in Emitter(plan).fw().source
    m1 = prebuild.plan_for('mamba1')                       # groups of 4 lanes, 16 staged steps: four kept steps per lane, not done
    assert m1.tile.L == 4 and Emitter(dataclasses.replace(m1, tile=dataclasses.replace(m1.tile, KS=3))).fw().source == Emitter(m1).fw().source
    # a traced RWKV-7 layer stages ten rows per timestep: 8 timesteps at four waves per workgroup, 16 at eight
    inputs, layer, _ = examples.build('rwkv7', 8, 1024, 4096, 128, 'meta', raw=True)
    lay = flex_rnn_amd.layer(layer)
    lay.graph(*[i.to(th.bfloat16) for i in inputs])
    call, = lay.calls
    lplan = planner.make_plan(call.fused.step, *call.metas)[0]
    assert lplan.tile.TS == 8 and lplan.tile.W == 4
    for v in launch.row_kernel_variants(lplan, False):
        assert v.TS == (16 if v.W == 8 else 8)
        planner.check_tile(v, lplan.H, lplan.NP, lplan.part)


def test_first_call_timing_skips_spilling_builds_and_reruns_close_contenders(tmp_path, monkeypatch):
    """`CompiledPlan._tune`: a build that spills more than `MAX_SPILL_BYTES` per lane is never launched (the first-ranked one
    aside), and candidates within 3 % of the fastest are run again by themselves and ranked by their medians."""
    from flex_rnn_amd import launch, prebuild
    from flex_rnn_amd.emit_hip import KernelSpec
    monkeypatch.setenv('FLEX_RNN_CACHE', str(tmp_path))
    monkeypatch.delenv('FLEX_RNN_RETUNE', raising=False)
    plan = prebuild.plan_for('rwkv7', (2, 64, 2, 128, 128))

    class Fake:
        _tune_rounds = 3
        _tune = launch.CompiledPlan._tune

        def __init__(self, spills, ms):
            self.plan, self.ms, self.launched, self.sel = plan, ms, [], None
            self.builds = {'frnn_bw2': [(KernelSpec('frnn_bw2', f'// build {i} {spills} {ms}', [], 64, ('1', '1', '1'), {}), None,
                                         {'scratch': s_, 'occupancy': 2, 'vgprs': 128}) for i, s_ in enumerate(spills)]}
            self._tune_pending, self.build_times, self.build_source = {'frnn_bw2'}, {}, {}

        def _capturing(self):
            return False

        def _device_name(self):
            return 'test-device'

        def _select(self, name, i):
            self.sel = i

        def _timed_launch(self, name, tensors):
            self.launched.append(self.sel)
            v = self.ms[self.sel]
            return v(len(self.launched)) if callable(v) else v

    f = Fake([0, 200, 20, 65], [3.0, 0.5, 2.0, 0.1])
    f._tune('frnn_bw2', {})
    assert set(f.launched) == {0, 2} and f.sel == 2 and f.build_times['frnn_bw2'][1] == float('inf')
    # two contenders within 3 %: the one with a single lucky run loses on the median
    lucky = iter([0.95] + [1.02] * 100)
    f = Fake([0, 0, 0], [1.0, lambda n: next(lucky), 1.5])
    f._tune('frnn_bw2', {})
    assert f.sel == 0 and f.launched.count(2) == 3 and f.launched.count(0) == 3 + 6 and f.launched.count(1) == 3 + 6
