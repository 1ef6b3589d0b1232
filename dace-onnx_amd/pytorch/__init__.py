from .module import DaceModule, dace_module, module_to_onnx, UnsupportedModule
