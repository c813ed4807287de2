"""The C++ mirror of the reference interface (include/nabla_optim.hpp,
include/nabla_checkpoint.hpp) replays the reference's own optimizer and trainer tests on
the device (tests/cpp/test_reference_kats.cpp)."""
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "test_reference_kats.bin")


def test_cpp_replay_is_built():
    assert os.path.exists(BIN), "build it with `make -C tests/cpp` (or __graft_entry__.build())"


def test_cpp_lr_at_step_matches_the_oracle_bit_for_bit():
    """The C++ mirror's lr_at_step over a grid of schedules and steps against the oracle's
    restatement of optim/core.rs:81-173 (no device involved)."""
    import struct

    import oracle as O

    r = subprocess.run([BIN, "--lr"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    scheds = [O.Schedule(0, 10, 110, 1e-5, 0.0), O.Schedule(0, 0, 7, 0.0, 0.0), O.Schedule(1, 5, 50, 0.0, 0.0),
              O.Schedule(1, 0, 1, 0.0, 0.0), O.Schedule(2, 0, 100, 1e-2, 0.3), O.Schedule(2, 0, 9, 0.5, 0.0),
              O.Schedule(3, 3, 0, 0.7, 0.0), O.Schedule(3, 0, 0, 0.5, 0.0),
              O.Schedule(0, 10, 5, 0.1, 0.0), O.Schedule(2, 0, 10, 1e-2, 1.5), O.Schedule(1, 40, 12, 0.0, 0.0)]
    lines = r.stdout.split("\n")[:-1]
    assert len(lines) == len(scheds) * 25
    for line in lines:
        k, step, bits = line.split()
        want = O.lr_at_step(scheds[int(k)], 3e-4, int(step))
        assert struct.pack("<d", want) == struct.pack("<Q", int(bits, 16)), line


@pytest.mark.gpu
def test_cpp_replay_of_reference_tests(gpu, tmp_path):
    r = subprocess.run([BIN, str(tmp_path)], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("ok    ") == 19 and "0 failure(s)" in r.stdout

    # the checkpoint the C++ side left behind is the one the Python mirror writes and reads
    from nabla_amd import checkpoint as ck
    from nabla_amd import optim as nb
    from nabla_amd.schedule import ScheduleState, Step
    import oracle as O
    from tests import helpers as H

    assert sorted(os.listdir(tmp_path)) == ["groups", "groups_mixed", "meta.txt", "mixed", "optim.nbla", "params.nbla"]
    shapes = [(1, 1), (1, 1)]
    opt = nb.Sgd.new(0.7, shapes, dtype="f64")
    scaler = nb.GradScaler.new()
    params, state, schedule = ck.load_checkpoint(str(tmp_path), opt, scaler)
    assert (state.epoch, state.step, state.grad_accum, state.rng_state) == (2, 3, 1, 42)
    assert schedule == ScheduleState(base_lr=0.1, schedule=Step(step_size=1, gamma=0.9))
    assert [(k, float(v[0, 0])) for k, v in params] == [("w", 1.5), ("b", -0.5)]
    assert opt.meta().lr == 0.1 and scaler.state().scale == 65536.0
    other = tmp_path / "py"
    ck.save_checkpoint(str(other), [("w", H.to_dev(np.array([1.5]), (1, 1))), ("b", H.to_dev(np.array([-0.5]), (1, 1)))],
                       nb.Sgd.new(0.1, shapes, dtype="f64"), nb.GradScaler.new(),
                       ScheduleState(base_lr=0.1, schedule=Step(step_size=1, gamma=0.9)),
                       ck.TrainState(epoch=2, step=3, grad_accum=1, rng_state=42))
    for name in ("meta.txt", "params.nbla", "optim.nbla"):
        assert (other / name).read_bytes() == (tmp_path / name).read_bytes(), name

    # and the GroupOptimizer checkpoint: meta.txt with the optim.group.* keys, optim.nbla with g{gi}. keys
    from nabla_amd import groups as G
    from nabla_amd.schedule import Cosine

    gdir = tmp_path / "groups"
    meta = (gdir / "meta.txt").read_text().splitlines()
    assert meta[:4] == ["version=1", "epoch=1", "step=2", "grad_accum=1"]
    assert meta[4:8] == ["optim.group.count=2", "optim.group.0.name=plain", "optim.group.0.kind=sgd", "optim.group.0.lr=0.5"]
    assert "optim.group.0.momentum=0.9" in meta and "optim.group.1.step_count=2" in meta and meta[-1] == "scaler.enabled=0"
    assert [n for n, _ in ck.load_tensors(str(gdir / "optim.nbla"))] == ["g0.v0", "g1.m0", "g1.v0"]
    w, b = H.to_dev(np.zeros(2), (1, 2)), H.to_dev(np.zeros(1), (1, 1))
    plain = G.ParamGroupConfig.sgd("plain", G.ParamSelector.Any([G.Suffix("bias")]), 0.5, 0.9, 0.0)
    decay = G.ParamGroupConfig.adamw("decay", G.ParamSelector.All(), 0.01, 0.1)
    gopt = G.GroupOptimizer.from_named_params([("l.weight", w), ("l.bias", b)], [plain], decay, dtype="f64")
    params, state, schedule = ck.load_checkpoint(str(gdir), gopt, None, into=[("l.weight", w), ("l.bias", b)])
    assert (state.epoch, state.step) == (1, 2) and schedule == ScheduleState(0.5, Cosine(1, 10, 0.0))
    assert gopt.group_optimizers()[1].step_count() == 2
    again = tmp_path / "groups_py"
    ck.save_checkpoint(str(again), [("l.weight", w), ("l.bias", b)], gopt, None, schedule,
                       ck.TrainState(epoch=1, step=2, grad_accum=1, rng_state=None), native=True)
    for name in ("meta.txt", "params.nbla", "optim.nbla"):
        assert (again / name).read_bytes() == (gdir / name).read_bytes(), name

    # and the mixed-precision checkpoint (f32 master weights as params.nbla): read by the Python
    # mirror, written again, the same bytes
    mdir = tmp_path / "mixed"
    mshapes = [(1, 8192 + 37), (1, 300)]
    mopt = nb.AdamW.new(1.0, mshapes, master=True)
    mscaler = nb.GradScaler.new()
    named = [("layer.w", H.dev_list([np.zeros(8192 + 37, np.uint16)], mshapes[:1])[0]),
             ("layer.b", H.dev_list([np.zeros(300, np.uint16)], mshapes[1:])[0])]
    _, mstate, msched = ck.load_checkpoint(str(mdir), mopt, mscaler, into=named)
    assert (mstate.step, msched) == (3, None) and mopt.step_count() == 3
    m = mopt.meta()
    assert (m.lr, m.beta2, m.weight_decay) == (2e-4, 0.95, 0.1)
    saved = dict(ck.load_tensors(str(mdir / "params.nbla")))
    for i, (name, p16) in enumerate(named):
        master = H.to_host(mopt.read_state(f"w{i}"))
        assert np.array_equal(saved[name].reshape(-1), master.astype(np.float64))
        H.assert_bits_equal([H.to_host(p16).reshape(-1)], [O.bf16_from_f32(master.reshape(-1))], "params narrowed from the master weights")
    mixed_again = tmp_path / "mixed_py"
    ck.save_checkpoint(str(mixed_again), named, mopt, mscaler, None, mstate)
    for name in ("meta.txt", "params.nbla", "optim.nbla"):
        assert (mixed_again / name).read_bytes() == (mdir / name).read_bytes(), name

    # and the GroupOptimizer whose groups keep master weights: params.nbla is every group's f32
    # master weights in the module's order; the Python mirror reads it, narrows the 16-bit tensors
    # from it and writes the same bytes again
    gm = tmp_path / "groups_mixed"
    gnames, gsizes = ["layer.w", "layer.bias", "layer.norm"], [8192 + 37, 300, 64]
    gnamed = [(n, H.dev_list([np.zeros(k, np.uint16)], [(1, k)])[0]) for n, k in zip(gnames, gsizes)]
    gopt2 = G.GroupOptimizer.adamw_with_decay_exclusions(gnamed, 1.0, 0.5, ["bias", "norm"], master=True)
    gscaler = nb.GradScaler.new()
    _, gstate, gsched = ck.load_checkpoint(str(gm), gopt2, gscaler, into=gnamed)
    assert (gstate.step, gsched) == (3, None) and [o.step_count() for o in gopt2.group_optimizers()] == [3, 3]
    assert [o.meta().weight_decay for o in gopt2.group_optimizers()] == [0.0, 0.1]
    saved = dict(ck.load_tensors(str(gm / "params.nbla")))
    assert list(saved) == gnames
    for idxs, o in zip(gopt2.group_indices(), gopt2.group_optimizers()):
        for k, i in enumerate(idxs):
            master = H.to_host(o.read_state(f"w{k}"))
            assert np.array_equal(saved[gnames[i]].reshape(-1), master.astype(np.float64))
            H.assert_bits_equal([H.to_host(gnamed[i][1]).reshape(-1)], [O.bf16_from_f32(master.reshape(-1))],
                                "group params narrowed from the master weights")
    gm_again = tmp_path / "groups_mixed_py"
    ck.save_checkpoint(str(gm_again), gnamed, gopt2, gscaler, None, gstate)
    for name in ("meta.txt", "params.nbla", "optim.nbla"):
        assert (gm_again / name).read_bytes() == (gm / name).read_bytes(), name
    # the whole file is checked before anything is written: an unknown key, a wrong shape
    bad_named = [("layer.w", gnamed[0][1]), ("layer.bias", gnamed[1][1]), ("other", gnamed[2][1])]
    with pytest.raises(ck.CheckpointError, match="unknown parameter key: layer.norm"):
        ck.load_checkpoint(str(gm), gopt2, gscaler, into=bad_named)
