"""Host logic of the Shampoo mirrors on the CPU (32-bit storage, as the reference forces there),
against vectors written by short runs of the reference's own optimizers."""
import numpy as np
import pytest
import torch

from optimizers import shampoo1 as S1
from optimizers import shampoo2 as S2
from optimizers.shampoo_common import BlockPartitioner

SHAPES = [(6, 10), (5,), (4, 1, 3), (9, 9)]


def close(got, want, tol=2e-5):
    got, want = torch.as_tensor(got).double(), torch.as_tensor(want).double()
    return float((got - want).norm()) <= tol * max(float(want.norm()), 1e-12)


def test_block_partitioner_shapes_and_round_trip():
    x = torch.arange(768 * 2304, dtype=torch.float32).reshape(768, 2304)
    part = BlockPartitioner(x, 1024)
    blocks = part.partition(x)
    assert [tuple(b.shape) for b in blocks] == [(768, 1024), (768, 1024), (768, 256)]
    assert part.shapes_for_preconditioners() == [[768, 768], [1024, 1024], [768, 768], [1024, 1024], [768, 768], [256, 256]]
    assert part.num_splits() == 2
    assert torch.equal(part.merge_partitions(blocks), x)
    y = torch.randn(7, 9)
    p2 = BlockPartitioner(y, 4)                       # 7 -> 4+3, 9 -> 4+4+1
    assert [tuple(b.shape) for b in p2.partition(y)] == [(4, 4), (4, 4), (4, 1), (3, 4), (3, 4), (3, 1)]
    assert torch.equal(p2.merge_partitions(p2.partition(y)), y)
    p3 = BlockPartitioner(y, 0)                       # 0 disables cutting
    assert len(p3.partition(y)) == 1 and p3.shapes_for_preconditioners() == [[7, 7], [9, 9]]
    p4 = BlockPartitioner(torch.zeros(8, 4), 4)       # exactly two pieces, no empty third
    assert [tuple(b.shape) for b in p4.partition(torch.zeros(8, 4))] == [(4, 4), (4, 4)]


@pytest.mark.parametrize("tag,mod,kw", [("s1", S1, {}), ("s2m0", S2, dict(inv_root_mode=0)), ("s2m1", S2, dict(inv_root_mode=1))])
def test_preconditioner_follows_reference_runs(golden, tag, mod, kw, tmp_path, monkeypatch):
    monkeypatch.chdir(tmp_path)                       # the eigenvalue log of shampoo2 lands in ./logs
    var = torch.from_numpy(golden["opt_init_0"]).clone()
    pre = mod.Preconditioner(var, {}, stat_decay=0.9, matrix_eps=1e-6, prec_maxorder=4, prec_bits=32, **kw)
    assert np.array_equal(np.array(pre._partitioner.shapes_for_preconditioners()), golden[f"pre_{tag}_shapes"])
    assert not pre.is_active()
    for st in range(3):
        grad = torch.from_numpy(golden[f"opt_grad_{st}_0"])
        torch.manual_seed(1000 + st)
        pre.add_statistics(grad)
        pre.compute_preconditioners()
        assert pre.is_active()
        assert close(pre.preconditioned_grad(grad), golden[f"pre_{tag}_out_{st}"]), (tag, st)
    for i, h in enumerate(pre.preconditioners):
        assert close(h.dequantize(), golden[f"pre_{tag}_prec_{i}"])
    if tag == "s1":
        for i, h in enumerate(pre.statistics):
            assert close(h.dequantize(), golden[f"pre_{tag}_stat_{i}"])
    if tag == "s2m0":
        assert (tmp_path / "logs").is_dir() and any((tmp_path / "logs").iterdir())


@pytest.mark.parametrize("tag,cls,kw", [
    ("adamw1", S1.ShampooAdamW, dict(lr=1e-2, weight_decay=0.05)),
    ("sgd1", S1.ShampooSGD, dict(lr=1e-2, momentum=0.9, weight_decay=1e-3, nesterov=True)),
    ("adamw2", S2.ShampooAdamW, dict(lr=1e-2, weight_decay=0.05, inv_root_mode=0)),
    ("sgd2", S2.ShampooSGD, dict(lr=1e-2, momentum=0.9, inv_root_mode=1))])
def test_optimizer_trajectories_follow_reference_runs(golden, tag, cls, kw, tmp_path, monkeypatch):
    monkeypatch.chdir(tmp_path)
    params = [torch.nn.Parameter(torch.from_numpy(golden[f"opt_init_{k}"]).clone()) for k in range(len(SHAPES))]
    opt = cls(params, start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2, stat_decay=0.9,
              prec_maxorder=4, prec_bits=32, **kw)
    for st in range(4):
        for k, p in enumerate(params):
            p.grad = torch.from_numpy(golden[f"opt_grad_{st}_{k}"]).clone()
        torch.manual_seed(2000 + st)
        opt.step()
    for k, p in enumerate(params):
        assert close(p.detach(), golden[f"opt_{tag}_final_{k}"]), (tag, k)


def test_vector_and_scalar_parameters_are_left_to_the_base_optimizer():
    pre = S1.Preconditioner(torch.zeros(5), {}, prec_bits=32)
    assert pre.statistics == [] and pre.preconditioners == []
    g = torch.randn(5)
    assert pre.preconditioned_grad(g) is g
    pre.add_statistics(g)
    pre.compute_preconditioners()
    assert pre.is_active()
    pre2 = S2.Preconditioner(torch.zeros(3, 1, 1), {}, prec_bits=32)
    assert pre2.statistics == []


def test_low_bit_request_on_cpu_stays_dense_and_state_dict_round_trips():
    params = [torch.nn.Parameter(torch.randn(80, 80))]
    opt = S1.ShampooAdamW(params, prec_bits=4, stat_compute_steps=1, prec_compute_steps=1, prec_maxorder=64)
    assert set(opt.name2qmap) == {"linear-2"} and opt.name2qmap["linear-2"].numel() == 16
    params[0].grad = torch.randn(80, 80)
    opt.step()
    pre = opt.state[params[0]]["preconditioner"]
    assert all(h.bits == 32 for h in pre.statistics + pre.preconditioners)       # CPU: never quantized
    assert len(pre.statistics) == 8                                             # 2 x 2 blocks, two sides each
    sd = opt.state_dict()
    opt2 = S1.ShampooAdamW(params, prec_bits=4, stat_compute_steps=1, prec_compute_steps=1, prec_maxorder=64)
    opt2.load_state_dict(sd)
    assert opt2.state[params[0]]["step"] == 1
    assert "Shampoo" in S1.ShampooSGD.__doc__ and "rect_t1" in S2.ShampooAdamW.__doc__


@pytest.mark.parametrize("mod,kw", [(S1, {}), (S2, dict(inv_root_mode=0)), (S2, dict(inv_root_mode=1))])
def test_checkpoint_holds_no_pickled_objects_and_resumes_bit_for_bit(mod, kw, tmp_path, monkeypatch):
    """state_dict() writes the preconditioners in their flat form (tensors, numbers, lists) under
    'shampoo_preconditioners', so torch.load(weights_only=True) reads the whole checkpoint (the reference pickles its
    Preconditioner objects, optimizers/shampoo2.py:311-317); a run resumed from it continues exactly like the
    uninterrupted one; a state that still holds the objects (the reference's form) loads as well."""
    import io
    monkeypatch.chdir(tmp_path)
    g = torch.Generator().manual_seed(3)
    shapes = [(12, 10), (7,), (9, 9)]
    init = [torch.randn(s, generator=g) for s in shapes]
    grads = [[torch.randn(s, generator=g) for s in shapes] for _ in range(6)]

    def make(params):
        return mod.ShampooAdamW(params, lr=1e-2, weight_decay=0.05, start_prec_step=2, stat_compute_steps=1, prec_compute_steps=2,
                                stat_decay=0.9, prec_maxorder=8, prec_bits=32, **kw)

    def run(opt, params, steps):
        for st in steps:
            for p, gr in zip(params, grads[st]):
                p.grad = gr.clone()
            torch.manual_seed(300 + st)
            opt.step()

    straight = [torch.nn.Parameter(t.clone()) for t in init]
    run(make(straight), straight, range(6))
    first = [torch.nn.Parameter(t.clone()) for t in init]
    opt = make(first)
    run(opt, first, range(3))
    sd = opt.state_dict()
    assert set(sd["shampoo_preconditioners"]) == {0, 1, 2}
    assert not any("preconditioner" in one for one in sd["state"].values())
    assert all("preconditioner" in opt.state[p] for p in first)                  # the live state keeps its objects
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True)
    resumed = [torch.nn.Parameter(p.detach().clone()) for p in first]
    opt2 = make(resumed)
    opt2.load_state_dict(loaded)
    assert opt2.state[resumed[0]]["preconditioner"].is_active()
    run(opt2, resumed, range(3, 6))
    for a, b in zip(straight, resumed):
        assert torch.equal(a.detach(), b.detach())
    # the reference's form: objects inside 'state'
    legacy = torch.optim.Optimizer.state_dict(opt)
    assert any("preconditioner" in one for one in legacy["state"].values())
    third = [torch.nn.Parameter(p.detach().clone()) for p in first]
    opt3 = make(third)
    opt3.load_state_dict(legacy)
    run(opt3, third, range(3, 6))
    for a, b in zip(straight, third):
        assert torch.equal(a.detach(), b.detach())
    # a flat state for another shape is refused
    other = make([torch.nn.Parameter(torch.zeros(20, 3))])
    bad = other.state_dict()
    bad["state"], bad["shampoo_preconditioners"] = {0: {"step": 1}}, {0: loaded["shampoo_preconditioners"][0]}
    with pytest.raises(ValueError):
        other.load_state_dict(bad)
