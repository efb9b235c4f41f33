"""Checkpoints in the reference's file format.

`cs::save(module, path)` (src/module/module.cpp:129-173) writes one Parquet file with two
columns, `key: string` (the qualified parameter name, e.g. "h.0.ln_1.weight") and
`value: list<item: float>` (the parameter flattened and widened to float32), one row per
parameter, a single row group.  `cs::load` (src/module/module.cpp:175-220) reads the rows back,
looks each key up in `named_parameters()` (an unknown key is an error), and copies
`tensor.to(parameter's dtype and device).view(parameter's shape)` into the parameter.

The reference leaves optimizer checkpoints unimplemented
(src/module/optimizer_module.cpp:45-51); `save_optimizer` / `load_optimizer` write AdamW's
first and second moments (and v_max) in the same layout under "<parameter>.m", ".v", ".v_max",
plus one row "<parameter>.t" holding the step count as two floats (t mod 2^24, t div 2^24, both
exact in float32), so that a run can resume with the state it stopped with.  The C++ host
library writes and reads the same files (cs::save / cs::load in csrc/host/src/checkpoint.cpp).

Everything here is host-side file work on torch tensors; nothing touches a kernel.
"""
from collections import OrderedDict

import pyarrow as pa
import pyarrow.parquet as pq
import torch

T_SPLIT = 1 << 24  # float32 holds every integer up to here

SCHEMA = pa.schema([pa.field("key", pa.utf8()), pa.field("value", pa.list_(pa.field("item", pa.float32())))])


def save_tensors(named_tensors, path):
    """named_tensors: mapping or iterable of (name, tensor).  Values are stored as float32."""
    items = list(named_tensors.items()) if hasattr(named_tensors, "items") else list(named_tensors)
    keys, offsets, chunks = [], [0], []
    for name, tensor in items:
        flat = tensor.detach().to("cpu", torch.float32).reshape(-1).contiguous().numpy()
        keys.append(name)
        chunks.append(pa.array(flat, type=pa.float32()))
        offsets.append(offsets[-1] + len(flat))
    values = pa.concat_arrays(chunks) if chunks else pa.array([], type=pa.float32())
    column = pa.ListArray.from_arrays(pa.array(offsets, type=pa.int32()), values,
                                      type=pa.list_(pa.field("item", pa.float32())))
    table = pa.Table.from_arrays([pa.array(keys, type=pa.utf8()), column], schema=SCHEMA)
    pq.write_table(table, path, row_group_size=max(1, len(keys)))


def load_tensors(path):
    """OrderedDict name -> flat float32 CPU tensor, in file order."""
    table = pq.read_table(path)
    if table.schema.names != ["key", "value"]:
        raise ValueError(f"not a parameter checkpoint: columns {table.schema.names}")
    out = OrderedDict()
    keys = table.column("key").to_pylist()
    column = table.column("value").combine_chunks()
    flat = column.flatten().to_numpy(zero_copy_only=False)
    offsets = column.offsets.to_numpy()
    for i, key in enumerate(keys):
        out[key] = torch.from_numpy(flat[offsets[i]:offsets[i + 1]].copy())
    return out


def load_into(named_parameters, path, assign=None):
    """Copies every row of the file into the parameter of the same name, converted to the
    parameter's dtype, device and shape.  A key the model does not have is an error, as in the
    reference; parameters the file does not mention are left alone.

    `assign(parameter, tensor)` does the copy; the default is `parameter.copy_(tensor)`."""
    params = dict(named_parameters.items() if hasattr(named_parameters, "items") else named_parameters)
    for key, flat in load_tensors(path).items():
        if key not in params:
            raise KeyError(f"wrong parameter name {key} in saved model")
        target = params[key]
        if assign is not None:
            assign(target, flat)
        else:
            if flat.numel() != target.numel():
                raise ValueError(f"{key}: {flat.numel()} values for a parameter of {target.numel()}")
            with torch.no_grad():
                target.copy_(flat.to(device=target.device, dtype=target.dtype).view(target.shape))


def save_optimizer(named_states, path):
    """named_states: iterable of (parameter name, state) where state has tensors m, v, optionally
    v_max (None when unused) and an integer t."""
    rows = []
    for name, state in named_states:
        rows.append((f"{name}.m", state["m"]))
        rows.append((f"{name}.v", state["v"]))
        if state.get("v_max") is not None:
            rows.append((f"{name}.v_max", state["v_max"]))
        t = int(state["t"])
        rows.append((f"{name}.t", torch.tensor([float(t % T_SPLIT), float(t // T_SPLIT)])))
    save_tensors(rows, path)


def load_optimizer(path):
    """name -> {"m", "v", "v_max" (or None), "t"} with flat float32 CPU tensors."""
    out = OrderedDict()
    for key, flat in load_tensors(path).items():
        name, _, field = key.rpartition(".")
        if field not in ("m", "v", "v_max", "t"):
            raise KeyError(f"not an optimizer checkpoint row: {key}")
        entry = out.setdefault(name, {"m": None, "v": None, "v_max": None, "t": 0})
        if field == "t":  # one value in files written before the count was split
            entry[field] = int(round(flat[0].item())) + (int(round(flat[1].item())) * T_SPLIT if flat.numel() > 1 else 0)
        else:
            entry[field] = flat
    return out
