from .linear import AWQW4A16Linear, SVDQW4A4Linear

__all__ = ["SVDQW4A4Linear", "AWQW4A16Linear"]
