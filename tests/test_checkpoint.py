"""The checkpoint file format of cs::save / cs::load (src/module/module.cpp:129-220): one Parquet
file, columns key: string and value: list<float>, one row per parameter.  test/test_load_save.cpp
saves a LayerNorm, zeroes its weight, loads and compares; the same round trip is done here on
plain tensors (no GPU needed) and, on the GPU, through the module layer."""
import os

import pyarrow.parquet as pq
import pytest
import torch

from core_scheduler_amd import checkpoint as ck


def test_file_layout_matches_the_reference(tmp_path):
    path = str(tmp_path / "model.parquet")
    params = {"ln.weight": torch.arange(6, dtype=torch.float32).reshape(2, 3), "ln.bias": torch.tensor([0.5, -1.0]),
              "empty": torch.zeros(0)}
    ck.save_tensors(params, path)
    table = pq.read_table(path)
    assert table.schema.names == ["key", "value"]
    assert str(table.schema.field("key").type) == "string"
    value_type = table.schema.field("value").type  # the inner field's name is the writer's business
    assert str(value_type).startswith("list<") and str(value_type.value_type) == "float"
    assert pq.ParquetFile(path).num_row_groups == 1  # WriteTable(..., chunk_size = number of parameters)
    assert table.column("key").to_pylist() == ["ln.weight", "ln.bias", "empty"]
    assert table.column("value").to_pylist() == [[0, 1, 2, 3, 4, 5], [0.5, -1.0], []]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16])
def test_round_trip_like_the_reference_test(tmp_path, dtype):
    # test/test_load_save.cpp:86-110 (float and double there; 16-bit storage widens exactly)
    path = str(tmp_path / "m.parquet")
    g = torch.Generator().manual_seed(1)
    weight = torch.randn(3 * 128, generator=g).to(dtype)
    bias = torch.randn(3 * 128, generator=g).to(dtype)
    ck.save_tensors([("weight", weight), ("bias", bias)], path)
    live = {"weight": torch.zeros_like(weight), "bias": torch.zeros(2, 192, dtype=dtype)}  # another view shape
    ck.load_into(live, path)
    if dtype == torch.float64:
        assert torch.allclose(live["weight"], weight)  # stored as float32, the reference's allclose bar
    else:
        assert torch.equal(live["weight"], weight)
        assert torch.equal(live["bias"].reshape(-1), bias)


def test_unknown_key_is_an_error_and_missing_ones_are_left_alone(tmp_path):
    path = str(tmp_path / "m.parquet")
    ck.save_tensors({"a": torch.ones(3)}, path)
    with pytest.raises(KeyError, match="wrong parameter name a"):
        ck.load_into({"b": torch.zeros(3)}, path)
    keep = {"a": torch.zeros(3), "c": torch.full((2,), 7.0)}
    ck.load_into(keep, path)
    assert torch.equal(keep["a"], torch.ones(3)) and torch.equal(keep["c"], torch.full((2,), 7.0))
    with pytest.raises(ValueError):
        ck.load_into({"a": torch.zeros(4)}, path)


def test_step_counts_beyond_float_precision_survive(tmp_path):
    path = str(tmp_path / "opt.parquet")
    t = (1 << 24) * 5 + 12345  # not representable in one float32
    ck.save_optimizer([("w", {"m": torch.zeros(2), "v": torch.zeros(2), "v_max": None, "t": t})], path)
    assert ck.load_optimizer(path)["w"]["t"] == t


def test_optimizer_state_round_trip(tmp_path):
    path = str(tmp_path / "opt.parquet")
    states = [("wte.weight", {"m": torch.randn(5, 4), "v": torch.rand(5, 4), "v_max": None, "t": 17}),
              ("ln_f.bias", {"m": torch.randn(4), "v": torch.rand(4), "v_max": torch.rand(4), "t": 17})]
    ck.save_optimizer(states, path)
    back = ck.load_optimizer(path)
    assert list(back) == ["wte.weight", "ln_f.bias"]
    for name, st in states:
        assert back[name]["t"] == 17
        assert torch.equal(back[name]["m"], st["m"].reshape(-1)) and torch.equal(back[name]["v"], st["v"].reshape(-1))
        assert (back[name]["v_max"] is None) == (st["v_max"] is None)


@pytest.mark.gpu
def test_module_tree_round_trip_on_the_gpu(tmp_path):
    from core_scheduler_amd import _cs_host as host

    sched = host.DynamicScheduler(0)
    root = host.Container()
    root.register_module("wte", host.EmbeddingModule(sched, 50, 16))
    h = root.register_module("h", host.Container())
    h.register_module("ln_1", host.LayerNormModule(sched, [16]))
    path = str(tmp_path / "gpu.parquet")
    before = {k: host.to_torch(sched, p).cpu() for k, p in root.named_parameters()}
    assert list(before) == ["wte.weight", "h.ln_1.weight", "h.ln_1.bias"]
    ck.save_tensors(before, path)
    for _, p in root.named_parameters():
        host.assign_(sched, p, torch.zeros(p.sizes()))
    assert all(host.to_torch(sched, p).abs().sum().item() == 0 for _, p in root.named_parameters())
    ck.load_into(dict(root.named_parameters()), path, assign=lambda p, flat: host.assign_(sched, p, flat))
    for k, p in root.named_parameters():
        assert torch.equal(host.to_torch(sched, p).cpu(), before[k]), k
    assert os.path.getsize(path) > 0


def _tree(host, sched):
    root = host.Container()
    root.register_module("wte", host.EmbeddingModule(sched, 50, 16))
    h = root.register_module("h", host.Container())
    h.register_module("ln_1", host.LayerNormModule(sched, [16]))
    return root


@pytest.mark.gpu
def test_cpp_save_is_read_by_python_and_python_files_by_cpp_load(tmp_path):
    """cs::save / cs::load (the C++ host library, Arrow C++) against checkpoint.py (pyarrow): either
    side reads what the other wrote, values bit-equal, same schema, one row group."""
    from core_scheduler_amd import _cs_host as host

    sched = host.DynamicScheduler(0)
    root = _tree(host, sched)
    before = {k: host.to_torch(sched, p).cpu() for k, p in root.named_parameters()}
    cpp_path, py_path = str(tmp_path / "cpp.parquet"), str(tmp_path / "py.parquet")
    host.save_module(root, cpp_path)
    table = pq.read_table(cpp_path)
    assert table.schema.names == ["key", "value"] and str(table.schema.field("key").type) == "string"
    assert str(table.schema.field("value").type.value_type) == "float"
    assert pq.ParquetFile(cpp_path).num_row_groups == 1
    read = ck.load_tensors(cpp_path)
    assert list(read) == list(before)
    for k in before:
        assert torch.equal(read[k], before[k].reshape(-1)), k
    # the other direction: Python writes other values, C++ loads them into the live module
    other = {k: torch.randn(v.shape, generator=torch.Generator().manual_seed(i)) for i, (k, v) in enumerate(before.items())}
    ck.save_tensors(other, py_path)
    host.load_module(root, py_path)
    for k, p in root.named_parameters():
        assert torch.equal(host.to_torch(sched, p).cpu(), other[k]), k
    # and C++ reads its own file back (test/test_load_save.cpp:86-110)
    host.load_module(root, cpp_path)
    for k, p in root.named_parameters():
        assert torch.equal(host.to_torch(sched, p).cpu(), before[k]), k


@pytest.mark.gpu
def test_cpp_optimizer_checkpoint_resumes_a_run(tmp_path):
    from core_scheduler_amd import _cs_host as host

    sched = host.DynamicScheduler(0)

    def run(steps, resume_from=None, save_to=None):
        torch.manual_seed(0)
        ln = host.LayerNormModule(sched, [32])
        opt = host.AdamWModule(sched, ln, lr=1e-2, amsgrad=True)
        if resume_from:
            host.load_module(ln, resume_from + ".model")
            host.load_optimizer(opt, resume_from + ".opt")
        for step in steps:
            g = torch.Generator().manual_seed(100 + step)
            x = host.from_torch(sched, torch.randn(8, 32, generator=g).to("cuda:0"))
            dy = host.from_torch(sched, torch.randn(8, 32, generator=g).to("cuda:0"))
            ln.forward(sched, x)
            ln.backward(sched, dy)
            opt.step(sched)
            opt.zero_grad(sched)
        if save_to:
            host.save_module(ln, save_to + ".model")
            host.save_optimizer(opt, save_to + ".opt")
        return ({k: host.to_torch(sched, p).cpu() for k, p in ln.named_parameters()},
                {k: (host.to_torch(sched, s.m).cpu(), s.t) for k, s in opt.named_states()})

    base = str(tmp_path / "ck")
    straight, st_straight = run(range(6))
    run(range(3), save_to=base)
    rows = ck.load_optimizer(base + ".opt")  # the Python side reads the C++ file
    assert set(rows) == {"weight", "bias"} and all(r["t"] == 3 and r["v_max"] is not None for r in rows.values())
    resumed, st_resumed = run(range(3, 6), resume_from=base)
    for k in straight:
        assert torch.equal(straight[k], resumed[k]), k
    for k in st_straight:
        assert st_straight[k][1] == st_resumed[k][1] == 6
        assert torch.equal(st_straight[k][0], st_resumed[k][0]), k
