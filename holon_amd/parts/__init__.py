"""The parts models are put together from. Importing this package registers the built-in ones."""
from .base import (FLOAT32, INT32, MODEL, Build, EmbedPart, NormPart, PagedState, ParamDecl, Part, PartialSums, SlotState,
                   Stream)
from .blocks import PreNorm
from .embed import Embedding, LMHead
from .ffn import DenseFFN, MoE, PolyNormFFN, SwiGLU
from .linear import Linear
from .mixers import GQA, ParallelMixers
from .norms import Normed, RMSNorm
from .positions import BandedRope, NoPosition, Rope, YarnRope, rope_table
from .convs import CausalConv
from .recurrent import DecayMemory, GatedDelta
from .sigmoid_attention import SigmoidWindowAttention
from .stream32 import LayerNorm, Pending, PreNorm32
from .dyt import DynamicTanh, Sandwich32, Scaled
from .softmax_attention import LatentAttention, SoftmaxAttention
from .mlstm import MLSTM
from .diff_attention import DiffAttention
from .parallel_block import Parallel32, RMSNorm32

__all__ = ["FLOAT32", "INT32", "MODEL", "Build", "EmbedPart", "NormPart", "PagedState", "ParamDecl", "Part", "PartialSums", "SlotState", "Stream", "PreNorm",
           "Embedding", "LMHead", "SwiGLU", "Linear", "GQA", "Normed", "RMSNorm", "NoPosition", "Rope", "rope_table", "BandedRope", "CausalConv", "DecayMemory", "GatedDelta",
           "SigmoidWindowAttention", "LayerNorm", "Pending", "PreNorm32", "ParallelMixers",
           "DynamicTanh", "Sandwich32", "Scaled", "LatentAttention", "SoftmaxAttention", "MLSTM", "YarnRope",
           "MoE", "PolyNormFFN", "Parallel32", "RMSNorm32", "DiffAttention", "DenseFFN"]
