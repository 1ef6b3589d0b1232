from .utils import torch_tensors_close, copy_to_gpu
