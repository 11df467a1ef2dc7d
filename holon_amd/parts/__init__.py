"""The parts models are put together from. Importing this package registers the built-in ones."""
from .base import (FLOAT32, INT32, MODEL, Build, EmbedPart, NormPart, PagedState, ParamDecl, Part, PartialSums, SlotState,
                   Stream)
from .blocks import PreNorm
from .embed import Embedding, LMHead
from .ffn import SwiGLU
from .linear import Linear
from .mixers import GQA
from .norms import Normed, RMSNorm
from .positions import NoPosition, Rope, rope_table

__all__ = ["FLOAT32", "INT32", "MODEL", "Build", "EmbedPart", "NormPart", "PagedState", "ParamDecl", "Part", "PartialSums", "SlotState", "Stream", "PreNorm",
           "Embedding", "LMHead", "SwiGLU", "Linear", "GQA", "Normed", "RMSNorm", "NoPosition", "Rope", "rope_table"]
