from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead
from .qwen3 import build_qwen3
from .bizipel import build_bizipel
from .kamivik import build_kamivik
from .repolix import build_repolix
from .nilepel import build_nilepel

__all__ = ["DecoderModel", "LayerRun", "TokenEmbedding", "OutputHead", "build_qwen3", "build_bizipel", "build_kamivik", "build_repolix", "build_nilepel"]
