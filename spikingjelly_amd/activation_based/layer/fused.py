"""Host-side glue between modules and the fused convolution / batch-norm / LIF kernels of
``hip_kernel/conv_bn_lif.py``: decides whether a ``conv -> BatchNorm -> LIFNode`` chain can run fused and, if so, runs
it and writes the neuron's state back.  Every function returns ``None`` when the chain has to run unfused (the caller
then calls its sub-modules one after the other, which gives the same result)."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ... import configure
from .. import neuron


def unobserved(*modules: Optional[nn.Module]) -> bool:
    """True when running ``modules`` as one fused kernel chain is indistinguishable from calling them one by one: none
    of them (and no global registration) has a forward, pre-forward or backward hook, which only ``Module.__call__``
    fires (output monitors, old-style ``weight_norm`` that rebuilds ``conv.weight`` in a pre-hook), and autocast is off
    (torch would run the convolution in the autocast dtype; the fused GEMMs keep fp32 operands)."""
    import torch.nn.modules.module as M

    if torch.is_autocast_enabled():
        return False
    for name in ("_global_forward_hooks", "_global_forward_pre_hooks", "_global_backward_hooks", "_global_backward_pre_hooks",
                 "_global_forward_hooks_always_called"):
        if len(getattr(M, name, ())):
            return False
    for m in modules:
        if m is None:
            continue
        for name in ("_forward_hooks", "_forward_pre_hooks", "_backward_hooks", "_backward_pre_hooks"):
            if len(getattr(m, name, ())):
                return False
    return True


def _pointwise(conv: nn.Module) -> bool:
    """A convolution that is one matrix product per position: kernel 1, stride 1, no padding, one group, no bias."""
    if not isinstance(conv, (nn.Conv1d, nn.Conv2d)):
        return False
    one = all(k == 1 for k in conv.kernel_size) and all(s == 1 for s in conv.stride) and all(d == 1 for d in conv.dilation)
    no_pad = all(p == 0 for p in conv.padding) if not isinstance(conv.padding, str) else conv.padding == "valid"
    return one and no_pad and conv.groups == 1 and conv.bias is None


def _bn_arguments(bn: nn.Module):
    """``(gamma, beta, (running_mean, running_var, batch_stats, momentum, eps, num_batches_tracked))`` the way
    ``_BatchNorm.forward`` derives them (``None`` for another kind of module).  The last element is the counter to
    increment (by the launch that updates the running statistics), or ``None``.  With ``momentum=None`` (cumulative
    moving average) the factor is ``1 / num_batches_tracked`` after the increment, which torch reads back to the host
    at this point of ``_BatchNorm.forward`` as well; the counter is then incremented here."""
    if not isinstance(bn, (nn.BatchNorm1d, nn.BatchNorm2d)):
        return None
    batch_stats = bn.training or (bn.running_mean is None and bn.running_var is None)
    update = bn.training and bn.track_running_stats
    tracked = bn.num_batches_tracked if update and bn.num_batches_tracked is not None else None
    momentum = float(bn.momentum or 0.0)
    if update and bn.momentum is None:
        if tracked is None or torch.compiler.is_compiling():  # (a value read back from the device is no part of a traced graph)
            return None
        tracked.add_(1)
        momentum = 1.0 / float(tracked)
        tracked = None
    if tracked is not None and not (tracked.is_cuda and tracked.dtype == torch.int64):
        tracked.add_(1)
        tracked = None
    running_mean = bn.running_mean if (update or not batch_stats) else None
    running_var = bn.running_var if (update or not batch_stats) else None
    return bn.weight, bn.bias, (running_mean, running_var, batch_stats, momentum, float(bn.eps), tracked)


def _lif_spec(node: nn.Module, x_like: torch.Tensor, need_grad: bool):
    from ..functional import neuron as F
    from ..hip_kernel import neuron_kernel as K
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = node.v_reset is None
    flags = K._flags(soft, node.detach_reset, getattr(node, "decay_input", False), F._hip_mode_flags(x_like))
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(node.surrogate_function) if need_grad else (0, 0.0)
    # (no time constant in the spec: an IF neuron has none, a parametric LIF's k travels as a tensor)
    tau = float(node.tau) if type(node) is neuron.LIFNode else 0.0
    return (tau, node.v_threshold, 0.0 if soft else float(node.v_reset), flags, sg_id, sg_alpha)


def _chain_neuron(node: nn.Module) -> bool:
    """The neuron at the end of a fused chain: an IF neuron, a plain or a parametric LIF."""
    return type(node) in (neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode)


def _neuron_k(node: nn.Module, x_like: torch.Tensor) -> Optional[torch.Tensor]:
    """``k = sigmoid(w)`` of a parametric LIF as the kernels read it (the sigmoid stays with autograd, which supplies
    ``dk/dw``; reference functional/neuron.py:2173-2182), ``None`` for a plain LIF."""
    if type(node) is not neuron.ParametricLIFNode:
        return None
    return node.w.sigmoid().to(device=x_like.device, dtype=torch.float32).reshape(1)


def _plain_hip_lif(node: nn.Module) -> bool:
    return (type(node) is neuron.LIFNode and node.backend == "hip" and node.step_mode == "m" and not node.store_v_seq)


def conv_bn_lif(x_seq: torch.Tensor, conv: Optional[nn.Module], bn: nn.Module, node: nn.Module, x_exact: bool = False,
                ssa: Optional[tuple] = None, attn: Optional[nn.Module] = None, container: Optional[nn.Module] = None
                ) -> Optional[torch.Tensor]:
    """``node(bn(conv(x_seq)))`` for ``x_seq [T, B, C, *positions]`` in one fused pass, or ``None``.

    ``conv is None``: ``x_seq`` already is the convolution output and only batch norm and the neuron are fused.
    ``ssa = (heads, scale)``: the spikes feed the spiking self-attention contraction bit-packed and the result is
    ``scale (V K^T) Q`` as ``[T, B, heads, channels_per_head, L]``.  With ``attn`` (the neuron that takes that result as
    its input) the result is ``attn``'s spikes instead, in the same shape, and ``None`` when ``attn`` cannot run inside
    the contraction.  ``x_exact``: ``x_seq`` holds values that bf16 represents exactly (spikes).  ``container``: the
    module through which the caller would otherwise call ``conv`` and ``bn`` (its hooks count like theirs)."""
    from ..hip_kernel import conv_bn_lif as C

    if not unobserved(conv, bn, node, attn, container):
        return None
    if (not configure.hip_fuse_conv_bn_lif or not _chain_neuron(node) or node.backend != "hip" or node.step_mode != "m"
            or node.store_v_seq or x_seq.dim() < 4):
        return None
    if attn is not None and (torch.compiler.is_compiling() or type(node) is not neuron.LIFNode):
        return None  # (the contraction with the attention's neuron inside: eager only, plain LIF in front of it)
    if conv is not None and (not _pointwise(conv) or x_seq.shape[2] != conv.in_channels):
        return None
    channels = conv.out_channels if conv is not None else x_seq.shape[2]
    if not isinstance(bn, (nn.BatchNorm1d, nn.BatchNorm2d)) or bn.num_features != channels:
        return None
    params = (p for p in (conv.weight if conv is not None else None, bn.weight, bn.bias, getattr(node, "w", None))
              if p is not None)
    need_grad = torch.is_grad_enabled() and (x_seq.requires_grad or any(p.requires_grad for p in params))
    x4 = x_seq.flatten(3)  # [T, B, C, L]
    if not C.supported(x4, need_grad):
        return None
    T, B, _, Lp = x4.shape
    if ssa is not None:
        from ..hip_kernel import attention_kernel as A

        heads, scale = ssa
        cph = channels // 3 // heads
        if channels != 3 * heads * cph or not A.ssa_packed_supported(x4.dtype, cph, Lp) or (B * channels * Lp) % 8 != 0:
            return None
        if attn is not None and (not configure.hip_fuse_ssa_lif or not _plain_hip_lif(attn)
                                 or not A.ssa_lif_supported(cph, Lp)):
            return None
    elif attn is not None:
        return None
    node._check_hip_surrogate()
    state_like = torch.empty((1,), dtype=x4.dtype, device=x4.device).expand(T, B, channels, *x_seq.shape[3:])
    (v,) = node.materialize_states((state_like,), (node.v,), "m")
    if need_grad and v.requires_grad:
        return None
    attn_v = None
    if attn is not None:
        attn._check_hip_surrogate()
        attn_like = torch.empty((1,), dtype=x4.dtype, device=x4.device).expand(T, B, heads, cph, Lp)
        (attn_v,) = attn.materialize_states((attn_like,), (attn.v,), "m")
        if need_grad and attn_v.requires_grad:
            return None
    bn_args = _bn_arguments(bn)  # (counts the batch: nothing below may give up)
    if bn_args is None:
        return None
    gamma, beta, bn_cfg = bn_args
    spec = _lif_spec(node, x4, need_grad)
    v3 = v.reshape(B, channels, Lp) if v.dim() != 3 else v
    out_shape = (T, B, channels, *x_seq.shape[3:])
    with torch.set_grad_enabled(need_grad):
        k = _neuron_k(node, x4)
        if conv is None:
            spikes, v_last = C.bn_lif(x4, gamma, beta, v3, bn_cfg, spec, k)
        elif ssa is None:
            spikes, v_last = C.conv_bn_lif(x4, conv.weight.view(channels, -1), gamma, beta, v3, bn_cfg, spec, x_exact, k)
        elif attn is None:
            out, v_last = C.conv_bn_lif_ssa(x4, conv.weight.view(channels, -1), gamma, beta, v3, bn_cfg, spec, x_exact,
                                            heads, cph, scale, k)
            node.v = v_last.reshape(out_shape[1:])
            return out.view(T, B, heads, cph, Lp)
        else:
            spikes, v_last, attn_v_last = C.conv_bn_lif_ssa_lif(
                x4, conv.weight.view(channels, -1), gamma, beta, v3, attn_v, bn_cfg, spec, x_exact, heads, cph, scale,
                _lif_spec(attn, x4, need_grad), need_grad)
            node.v = v_last.reshape(out_shape[1:])
            attn.v = attn_v_last
            return spikes
    node.v = v_last.reshape(out_shape[1:])
    return spikes.view(out_shape)


def lif_conv_bn_lif(pre_seq: torch.Tensor, pre_node: nn.Module, conv: nn.Module, bn: nn.Module, node: nn.Module,
                    container: Optional[nn.Module] = None) -> Optional[torch.Tensor]:
    """``node(bn(conv(pre_node(pre_seq))))`` for ``pre_seq [T, B, C, *positions]`` (or ``[T, B, heads, C / heads, L]``,
    as the attention's neuron sees it: its state keeps that shape) in one autograd node whose first
    neuron writes its spikes bit-packed and whose convolution reads them as bits (the spikes never exist as a float
    tensor), or ``None`` when the chain does not qualify (the caller then runs the modules one by one).  This is the
    ``attn_lif -> proj_conv -> proj_bn -> proj_lif`` tail of the reference's ``SpikingSelfAttention.forward``
    (layer/attention.py:376-384)."""
    from ..functional import neuron as F
    from ..hip_kernel import conv_bn_lif as C

    if not unobserved(pre_node, conv, bn, node, container):
        return None
    if (not configure.hip_fuse_conv_bn_lif or not getattr(configure, "hip_conv_bit_spikes", True)
            or not _chain_neuron(node) or node.backend != "hip" or node.step_mode != "m" or node.store_v_seq
            or not _plain_hip_lif(pre_node) or pre_seq.dim() < 4):
        return None
    Cin = conv.in_channels
    if not _pointwise(conv) or pre_seq.numel() == 0:
        return None
    if pre_seq.shape[2] == Cin:
        positions = tuple(pre_seq.shape[3:])
    elif pre_seq.dim() == 5 and pre_seq.shape[2] * pre_seq.shape[3] == Cin:
        positions = (pre_seq.shape[4],)
    else:
        return None
    channels = conv.out_channels
    if not isinstance(bn, (nn.BatchNorm1d, nn.BatchNorm2d)) or bn.num_features != channels:
        return None
    params = (p for p in (conv.weight, bn.weight, bn.bias, getattr(node, "w", None)) if p is not None)
    need_grad = torch.is_grad_enabled() and (pre_seq.requires_grad or any(p.requires_grad for p in params))
    x4 = pre_seq.reshape(pre_seq.shape[0], pre_seq.shape[1], Cin, -1)  # [T, B, Cin, L]
    T, B, _, Lp = x4.shape
    if not C.lif_conv_bn_lif_supported(x4, need_grad) or (B * Cin * Lp) % 8 != 0:
        return None
    if need_grad and not F._hip_recompute(x4.flatten(1)):
        return None  # the first neuron's backward replays its forward
    node._check_hip_surrogate()
    pre_node._check_hip_surrogate()
    (pre_v,) = pre_node.materialize_states((pre_seq,), (pre_node.v,), "m")
    state_like = torch.empty((1,), dtype=x4.dtype, device=x4.device).expand(T, B, channels, *positions)
    (v,) = node.materialize_states((state_like,), (node.v,), "m")
    if need_grad and (v.requires_grad or pre_v.requires_grad):
        return None
    bn_args = _bn_arguments(bn)  # (counts the batch: nothing below may give up)
    if bn_args is None:
        return None
    gamma, beta, bn_cfg = bn_args
    v3 = v.reshape(B, channels, Lp) if v.dim() != 3 else v
    pre_v3 = pre_v.reshape(B, Cin, Lp)
    with torch.set_grad_enabled(need_grad):
        spikes, v_last, pre_v_last = C.lif_conv_bn_lif(x4, pre_v3, conv.weight.view(channels, -1), gamma, beta, v3, bn_cfg,
                                                       _lif_spec(pre_node, x4, need_grad), _lif_spec(node, x4, need_grad),
                                                       _neuron_k(node, x4))
    node.v = v_last.reshape(B, channels, *positions)
    pre_node.v = pre_v_last.reshape(pre_seq.shape[1:])
    return spikes.view(T, B, channels, *positions)

