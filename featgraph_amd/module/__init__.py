from .spmm import VanillaSpMMhip, VanillaSpMMx86, VanillaSpMMcuda
from .sddmm import VanillaSDDMMhip, VanillaSDDMMx86, VanillaSDDMMcuda, MultiHeadSDDMMhip, GSDDMMhip
from .gspmm import GSpMMhip
from .common import placeholder
from .softmax import EdgeSoftmaxhip, EdgeSoftmaxSpMMhip
from .attention import GraphAttentionhip
