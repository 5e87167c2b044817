from .micro_adam import MicroAdam

__all__ = [
    'MicroAdam',
]
