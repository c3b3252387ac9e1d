from . import pshattn

__all__ = ["pshattn"]
