from .cumsum import cumsum

__all__ = ["cumsum"]
