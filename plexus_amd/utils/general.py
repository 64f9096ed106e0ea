"""Helpers of the path that the reference keeps in plexus/utils/general.py."""
import random

import numpy as np
import torch


def set_seed(seed=0):
    """plexus/utils/general.py:9-13 -- seed every generator the path may draw from."""
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


def pad_dimension(dim_value, num_gpus, second_num_gpus=1):
    """plexus/utils/general.py:20-23 -- smallest multiple of num_gpus * second_num_gpus >= dim_value."""
    prod_num_gpus = num_gpus * second_num_gpus
    remainder = dim_value % prod_num_gpus
    return dim_value if remainder == 0 else dim_value + prod_num_gpus - remainder


def analyze_csr_tensor(sparse_tensor):
    """plexus/utils/general.py:52-73 -- (number of stored values, Frobenius norm)."""
    values = sparse_tensor.val if hasattr(sparse_tensor, "val") else sparse_tensor.values()
    return values.numel(), torch.sqrt(torch.sum(values**2)).item()
