"""Connector-name helpers (``daceml/onnx/nodes/node_utils.py``)."""
import typing


def parse_variadic_param(param: str) -> typing.Tuple[str, int]:
    """Split ``"name__3"`` into ``("name", 3)``."""
    split = param.split('__')
    if len(split) != 2:
        raise ValueError("Unable to parse variadic parameter '{}'".format(param))
    name, number = split
    if number[0] == '0' and len(number) > 1:
        raise ValueError("Variadic parameters must not be numbered with leading zeroes, got: '{}'".format(number))
    number = int(number)
    if number < 0:
        raise ValueError("Variadic parameters numberings must be greater than zero, got: '{}'".format(number))
    return name, number
