from .bmm_chain import (BatchGemmGemm, BatchGemmGemmMMA, BatchGemmSoftmaxGemm,
                        BatchGemmSoftmaxGemmMMA)
from .conv_chain import (Conv1x1Conv1x1, Conv1x1Conv3x3, Conv1x1ReluConv3x3, Conv3x3Conv1x1, Conv3x3ReluConv1x1,
                         Depthwise3x3Conv1x1, conv_chain, conv_relu_conv)
from .elementwise import ACT_KINDS, ELEM_KINDS, ReLU, activation, elementwise
