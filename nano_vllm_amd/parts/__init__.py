from .spec import PartSpec, LayerSpec, LayerRun, ModelSpec, PagedKV, FixedState
from .base import Part, ParamDecl, Source, BuildContext
from .registry import register_part, make_part, known_parts
from .model import Model, LayerCache, torch_dtype

__all__ = ["PartSpec", "LayerSpec", "LayerRun", "ModelSpec", "PagedKV", "FixedState", "Part", "ParamDecl",
           "Source", "BuildContext", "register_part", "make_part", "known_parts", "Model", "LayerCache",
           "torch_dtype"]
