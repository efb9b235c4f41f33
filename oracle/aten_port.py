"""TEST INFRASTRUCTURE ONLY: the reference's op sequences on the ATen CPU backend.

Each function issues the same ATen calls, in the same order and with the same
arguments, as one reference task body (cited per function), to the CPU
kernels of the installed torch.  libtorch is the library the reference links
(env.yaml:182 pins 2.3.1; this image has a later release of the same ops).
It serves two purposes: it pins the C oracle, and it is the CPU baseline the
benchmark times next to the GPU kernels.

Storage rule for 16-bit inputs: widen to float32 first and round once at the
end, which is what the reference's AMP tests compare against
(test/test_cross_entropy.cpp:125-127).
"""
import torch

aten = torch.ops.aten


def cross_entropy_forward(x, target, ignore_index=-100, reduction=1, weight=None):
    """src/compute/cross_entropy.cpp:57-63 -> (log_probs, loss, total_weight); `weight` as :52-55"""
    log_probs = aten.log_softmax(x, 1)
    loss, total_weight = aten.nll_loss_forward(log_probs, target, weight, reduction, ignore_index)
    return log_probs, loss, total_weight


def cross_entropy_backward(log_probs, loss, target, total_weight, ignore_index=-100, reduction=1, weight=None):
    """src/compute/cross_entropy.cpp:97-109 -> grad_input"""
    dnll = aten.nll_loss_backward(torch.ones_like(loss), log_probs, target, weight, reduction, ignore_index,
                                  total_weight)
    return aten._log_softmax_backward_data(dnll, log_probs, 1, log_probs.dtype)


def cross_entropy(x, target, ignore_index=-100, reduction=1, weight=None):
    """forward then backward, as example/gpt2/gpt2_single_device.cpp:674,693-694"""
    lp, loss, tw = cross_entropy_forward(x, target, ignore_index, reduction, weight)
    return loss, cross_entropy_backward(lp, loss, target, tw, ignore_index, reduction, weight), tw


def embedding_forward(weight, indices, padding_idx=-1):
    """src/compute/embedding.cpp:117-121"""
    return aten.embedding(weight, indices.view(-1, indices.size(-1)), padding_idx, False, False)


def embedding_backward(grad_output, indices, num_weights, padding_idx=-1, scale_grad_by_freq=False):
    """src/compute/embedding.cpp:147-157 (the `=` branch); `sparse` stays false"""
    return aten.embedding_backward(grad_output, indices, num_weights, padding_idx, scale_grad_by_freq, False)


def token_position_forward(wte, wpe, ids):
    """example/gpt2/gpt2_single_device.cpp:541-545"""
    T = ids.size(-1)
    pos = torch.arange(T, dtype=torch.int64)
    tok = embedding_forward(wte, ids)
    pe = embedding_forward(wpe, pos.view(1, T))
    return tok + pe.broadcast_to(tok.shape)


def token_position_backward(dout, ids, V):
    """example/gpt2/gpt2_single_device.cpp:565-567 -> (dwte, dwpe)"""
    T = ids.size(-1)
    pos = torch.arange(T, dtype=torch.int64)
    dwpe = embedding_backward(dout.sum(0), pos, T)
    dwte = embedding_backward(dout, ids, V)
    return dwte, dwpe


def layernorm_forward(x, gamma, beta, eps=1e-5):
    """src/compute/layer_norm.cpp:163-169 -> (y, mean, rstd)"""
    return aten.native_layer_norm(x, [x.size(-1)], gamma, beta, eps)


def layernorm_backward(dy, x, mean, rstd, gamma, beta):
    """src/compute/layer_norm.cpp:263-266 and :321-324 -> (dx, dgamma, dbeta)

    The reference calls native_layer_norm_backward twice with masks {1,0,0}
    and {0,1,1}; so does this."""
    dx, _, _ = aten.native_layer_norm_backward(dy, x, [x.size(-1)], mean, rstd, gamma, beta,
                                               [True, False, False])
    _, dg, db = aten.native_layer_norm_backward(dy, x, [x.size(-1)], mean, rstd, gamma, beta,
                                                [False, True, beta is not None])
    return dx, dg, db


def gelu_forward(x, approximate="none"):
    """src/compute/gelu.cpp:39 (approximate is always "none" there)"""
    return aten.gelu(x, approximate=approximate)


def gelu_backward(dy, x, approximate="none"):
    """src/compute/gelu.cpp:61-62"""
    return aten.gelu_backward(dy, x, approximate=approximate)
