from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

__all__ = ["LayerSpec", "ModelSpec", "PartSpec", "RunSpec"]
