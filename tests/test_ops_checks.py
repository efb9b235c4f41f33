"""Argument checks of core_scheduler_amd.ops that run before anything touches a device.

The kernels take one element type and one element count for a parameter, its gradient and its
optimizer state, and add into an existing embedding gradient with the incoming gradient's type
and row length; a mismatch must raise instead of reading or writing past a buffer.
"""
import pytest
import torch

from core_scheduler_amd import ops

HP = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, t=1)


@pytest.mark.parametrize("which", ["dw", "m", "v", "v_max"])
@pytest.mark.parametrize("fault", ["dtype", "numel"])
def test_adamw_step_rejects_mismatched_tensors(which, fault):
    t = {k: torch.zeros(16) for k in ("w", "dw", "m", "v", "v_max")}
    t[which] = torch.zeros(16, dtype=torch.bfloat16) if fault == "dtype" else torch.zeros(8)
    with pytest.raises(ValueError, match="AdamW"):
        ops.adamw_step(t["w"], t["dw"], t["m"], t["v"], v_max=t["v_max"], **HP)


def test_multi_tensor_adamw_rejects_mixed_parameter_dtypes():
    with pytest.raises(ValueError, match="one dtype"):
        ops.MultiTensorAdamW([torch.zeros(4), torch.zeros(4, dtype=torch.bfloat16)],
                             [torch.zeros(4), torch.zeros(4, dtype=torch.bfloat16)])


@pytest.mark.parametrize("bad", [torch.zeros(10, 8, dtype=torch.float64), torch.zeros(10, 4), torch.zeros(9, 8)])
def test_embedding_backward_rejects_a_gradient_of_another_type_or_shape(bad):
    dout, ids = torch.zeros(4, 8), torch.zeros(4, dtype=torch.int64)
    with pytest.raises(ValueError, match="dweight"):
        ops.embedding_backward(dout, ids, 10, dweight=bad)
    with pytest.raises(ValueError, match="dwte"):
        ops.embedding_backward_fused(dout.reshape(1, 4, 8), ids.reshape(1, 4), 10, dwte=bad, dwpe=torch.zeros(4, 8))


def test_ops_refuse_cpu_tensors():
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.gelu_forward(torch.zeros(8))
