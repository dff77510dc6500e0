"""Blocked (tiled + permuted) parameter layouts.

Same public surface as the reference's
``src/tpp_pytorch_extension/utils/blocked_layout.py`` for the pieces the
quantized-linear path touches: ``BlockingManager`` (:28-92), ``BlockedParameter``
(:248-306) and ``BlockedModule`` (:308-364, state-dict round trip through the
plain layout).  The blocked layout is what the quantizers take as input:
``W[N, K]`` viewed as ``[N/bk, bk, K/bc, bc/v, v]`` and permuted to
``[N/bk, K/bc, bc/v, bk, v]``.
"""
import torch

from . import float8  # noqa: F401  (installs Tensor.cvt_to)


def _split_sizes(extent, factors):
    """View sizes of one dimension blocked by `factors` (None, int or list)."""
    if factors is None:
        return [extent]
    if isinstance(factors, int):
        factors = [factors]
    elif not isinstance(factors, (list, tuple)):
        raise ValueError("Unsupported blocking factor: %s" % (factors,))
    inner = 1
    for f in factors:
        inner *= f
    if extent % inner != 0:
        raise AssertionError(
            "Blocking factor doesn't divide dim evenly shape = %s, BF = %s" % (extent, factors)
        )
    return [extent // inner] + list(factors)


class BlockingManager(object):
    """view + permute description of a blocked layout and its inverse."""

    def __init__(self, orig_shape, blocking_factors=None, permute=None):
        ndim = len(orig_shape)
        if blocking_factors is None:
            blocking_factors = [None] * ndim
        assert len(blocking_factors) == ndim
        self.orig_shape = orig_shape
        view = []
        for extent, factors in zip(orig_shape, blocking_factors):
            view.extend(_split_sizes(extent, factors))
        self.view_shape = view
        self.permute = permute
        if permute is None:
            self.back_permute = None
            self.blocked_shape = view
        else:
            assert isinstance(permute, (list, tuple)) and sorted(permute) == list(range(len(view)))
            inverse = [0] * len(permute)
            for dst, src in enumerate(permute):
                inverse[src] = dst
            self.back_permute = inverse
            self.blocked_shape = [view[src] for src in permute]

    def block(self, input):
        assert input.shape == self.orig_shape
        out = input.view(self.view_shape)
        return out.permute(self.permute).contiguous() if self.permute else out

    def unblock(self, input):
        assert list(input.shape) == self.blocked_shape, "Shapes: %s, %s" % (input.shape, self.blocked_shape)
        out = input.permute(self.back_permute).contiguous() if self.back_permute else input
        return out.view(self.orig_shape)


class BlockedParameter(torch.nn.Parameter):
    """A Parameter that can switch between its plain and its blocked layout."""

    def __new__(cls, data=None, requires_grad=True, **kwargs):
        return super(BlockedParameter, cls).__new__(cls, data=data, requires_grad=requires_grad)

    def __init__(self, *args, **kwargs):
        self.blocked = False
        self.blocking_param = None
        self.blocking_manager = None

    def set_blocking_param(self, blocking_param):
        self.blocking_param = blocking_param

    def is_blocked(self):
        return self.blocked

    def _ensure_manager(self):
        if self.blocking_manager is not None:
            return True
        if self.blocking_param is None:
            return False
        bp = self.blocking_param
        self.unblocked_dtype = self.dtype
        self.blocked_dtype = bp[2] if (len(bp) > 2 and bp[2] is not None) else self.dtype
        self.blocking_manager = BlockingManager(self.data.shape, blocking_factors=bp[0], permute=bp[1])
        return True

    def block(self):
        if self.blocked or not self._ensure_manager():
            return
        if self.blocked_dtype == torch.uint8:
            self.requires_grad_(False)
        self.data = self.blocking_manager.block(self.data).cvt_to(self.blocked_dtype)
        if self.grad is not None:
            self.grad.data = self.blocking_manager.block(self.grad.data).cvt_to(self.blocked_dtype)
        self.blocked = True

    def unblock(self):
        if not self.blocked:
            return
        self.data = self.blocking_manager.unblock(self.data).cvt_to(self.unblocked_dtype)
        if self.grad is not None:
            self.grad.data = self.blocking_manager.unblock(self.grad.data).cvt_to(self.unblocked_dtype)
        self.blocked = False


class BlockedModule(torch.nn.Module):
    """Saves / loads its BlockedParameters in the plain layout."""

    def _blocked_params(self):
        return [(n, p) for n, p in self.named_parameters(recurse=False)
                if isinstance(p, BlockedParameter) and p.is_blocked()]

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        touched = self._blocked_params()
        for _, p in touched:
            p.unblock()
        super(BlockedModule, self)._save_to_state_dict(destination, prefix, keep_vars)
        for _, p in touched:
            p.block()

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                              unexpected_keys, error_msgs):
        assign = local_metadata.get("assign_to_params_buffers", False)
        reblock, rewrap = [], {}
        for n, p in self.named_parameters(recurse=False):
            if isinstance(p, BlockedParameter):
                if p.is_blocked():
                    p.unblock()
                    reblock.append(n)
                if p.is_meta or assign:
                    rewrap[n] = getattr(p, "blocking_param", None)
        super(BlockedModule, self)._load_from_state_dict(
            state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)
        for n, bp in rewrap.items():
            fresh = BlockedParameter(getattr(self, n).data)
            fresh.set_blocking_param(bp)
            setattr(self, n, fresh)
        for n in reblock:
            p = getattr(self, n)
            if isinstance(p, BlockedParameter):
                p.block()


def block_model_params(model):
    for m in model.modules():
        if hasattr(m, "maybe_block_params"):
            m.maybe_block_params()
