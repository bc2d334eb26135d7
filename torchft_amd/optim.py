"""Optimizer gate for the DDP flow (torchft/optim.py:24-63): ``zero_grad`` opens the
step by starting the quorum, ``step`` only applies the update if the replica group
voted to commit.  No arithmetic of its own; everything else is the wrapped optimizer's."""

from __future__ import annotations

from typing import TYPE_CHECKING, Callable, Optional

from torch.optim import Optimizer

if TYPE_CHECKING:
    from .manager import Manager


def _delegate(name: str) -> Callable:
    def call(self: "OptimizerWrapper", *args: object, **kwargs: object) -> object:
        return getattr(self.optim, name)(*args, **kwargs)

    call.__name__ = name
    call.__doc__ = f"``{name}`` of the wrapped optimizer."
    return call


class OptimizerWrapper(Optimizer):
    """``OptimizerWrapper(manager, optim)``: use it wherever the plain optimizer was used.
    It is an ``Optimizer`` (schedulers accept it) but owns no state: ``param_groups``,
    ``state``, ``state_dict`` / ``load_state_dict`` / ``add_param_group`` are the wrapped
    optimizer's."""

    def __init__(self, manager: "Manager", optim: Optimizer) -> None:  # no Optimizer.__init__
        self.manager = manager
        self.optim = optim

    param_groups = property(lambda self: self.optim.param_groups)  # type: ignore[assignment]
    state = property(lambda self: self.optim.state)  # type: ignore[assignment]
    add_param_group = _delegate("add_param_group")
    load_state_dict = _delegate("load_state_dict")
    state_dict = _delegate("state_dict")

    def zero_grad(self, set_to_none: bool = True) -> None:
        """A new step begins: the quorum is started (and runs alongside the forward pass)."""
        self.manager.start_quorum()
        self.optim.zero_grad(set_to_none)

    def step(self, closure: Optional[object] = None) -> None:
        """Applies the update only if the group commits this step."""
        assert closure is None, "optimizers that use closures are not supported"
        if self.manager.should_commit():
            self.optim.step()
