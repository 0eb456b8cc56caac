from .sddmm import VanillaSDDMMhip, MultiHeadSDDMMhip
from .spmm import VanillaSpMMhip, MultiHeadSpMMhip
from .general import GeneralizedSpMMhip, GeneralizedSDDMMhip, VanillaSpMMGradhip
from .softmax import EdgeSoftmaxhip, MultiHeadSDDMMSoftmaxhip
from .attention import MultiHeadAttentionhip
from .general import MultiHeadGeneralizedSpMMhip
from .backward import (EdgeSoftmaxGradhip, MultiHeadAttentionGradhip, MultiHeadSDDMMGradhip,
                       MultiHeadSpMMGradhip)
