"""``ONNXForward``: the plugin interface for expansions of ONNX library nodes.

Same contract as ``daceml/onnx/forward_implementation_abc.py:11-51``: subclasses
give two static methods, ``forward_can_be_applied(node, state, sdfg) -> bool``
(default ``True``) and ``forward(node, state, sdfg)`` returning a node or an
SDFG, and are registered with keyword arguments ``op`` (ONNX op name) and
``name`` (implementation name). The reference gets its registry from
``dace.registry.make_registry``; the few lines of it that are used
(``register`` / ``extensions``) are provided here.
"""
import abc
import typing

from ..sdfg import SDFG, SDFGState, Node


class ONNXForward(abc.ABC):
    """ABC for ONNX op forward implementations.

    ``register`` expects ``op`` (the ONNX op name) and ``name`` (the implementation name).
    """
    _registry_: typing.Dict[type, typing.Dict[str, typing.Any]] = {}

    @classmethod
    def register(cls, subclass, **kwargs):
        cls._registry_[subclass] = kwargs
        if "op" in kwargs and "name" in kwargs:
            # bind right away so that implementations defined after the node
            # classes exist become selectable (the reference binds once, at
            # import time, onnx_op.py:646-687)
            from .nodes.onnx_op import bind_implementation
            bind_implementation(kwargs["op"], kwargs["name"], subclass)

    @classmethod
    def unregister(cls, subclass):
        cls._registry_.pop(subclass, None)

    @classmethod
    def extensions(cls) -> typing.Dict[type, typing.Dict[str, typing.Any]]:
        return cls._registry_

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        """Return whether this expansion can be applied to ``node``."""
        return True

    @staticmethod
    @abc.abstractmethod
    def forward(node, state: SDFGState, sdfg: SDFG) -> typing.Union[Node, SDFG]:
        """Expand ``node`` and return its expansion."""
        ...

    @classmethod
    def registered_implementations(cls, op_name: str) -> typing.List[typing.Tuple[str, "ONNXForward"]]:
        impls = []
        for impl, args in cls.extensions().items():
            if "op" in args and args["op"] == op_name:
                impls.append((args["name"], impl))
        return impls
