from .spmm import VanillaSpMMhip, VanillaSpMMx86, VanillaSpMMcuda
from .sddmm import VanillaSDDMMhip, VanillaSDDMMx86, VanillaSDDMMcuda, MultiHeadSDDMMhip
from .gspmm import GSpMMhip
from .common import placeholder
