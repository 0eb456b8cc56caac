from .sddmm import VanillaSDDMMhip, MultiHeadSDDMMhip
from .spmm import VanillaSpMMhip, MultiHeadSpMMhip
