from .base_model import BaseModel, HFBaseModel, HFDecBaseModel

__all__ = ["BaseModel", "HFBaseModel", "HFDecBaseModel"]
