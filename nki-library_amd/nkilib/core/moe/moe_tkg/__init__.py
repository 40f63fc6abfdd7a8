from .moe_tkg import moe_tkg

__all__ = ["moe_tkg"]
