from .micro_adam import *
