import torch

QuantTensor = tuple[torch.Tensor, torch.Tensor]
