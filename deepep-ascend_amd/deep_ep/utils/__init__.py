from . import event, math, semantic
