from . import ops, build
