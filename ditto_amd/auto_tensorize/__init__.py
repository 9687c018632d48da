"""Chain descriptors of the hyper_fusion path (reference: python/ditto/auto_tensorize)."""
from .hyper_fusion import (ChainSchedule, CPUTensorizeParam, CUDATensorizeParam, FusionChoice, MatchInfo,
                           TensorizeHyperFusionState, build_cpu_tensorize_param, build_fusion_choice,
                           cuda_tensorize_param, fusion_choice, match_info, tensorize_cpu, tensorize_cuda,
                           tensorize_hip, tensorize_hyper_fusion_state)
from .intrinsic import PackedIntrinsic, cpu_intrin, cuda_wmma, hip_mfma, intrinsic_match, packed_intrinsic
from .pattern import (PATTERN_ALLRED, PATTERN_CUBIC, PATTERN_LOCAL, PATTERN_SHUFFLE, GetOpPattern, IsAllred,
                      IsCubic, IsLocal, IsShuffle)
from .state import FusionContext, SerialFusionState, build_fusion_context, build_serial_fusion_state, validate
