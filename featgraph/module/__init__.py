from featgraph_amd.module import (VanillaSpMMhip, VanillaSpMMx86, VanillaSpMMcuda,
                                  VanillaSDDMMhip, VanillaSDDMMx86, VanillaSDDMMcuda,
                                  MultiHeadSDDMMhip, GSpMMhip, GSDDMMhip, EdgeSoftmaxhip,
                                  EdgeSoftmaxSpMMhip, GraphAttentionhip, placeholder)
