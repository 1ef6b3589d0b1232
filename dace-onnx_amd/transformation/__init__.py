from .fusion import fuse_onnx_graph  # noqa: F401
