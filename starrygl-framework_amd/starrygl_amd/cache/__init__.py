from .NodeState import DistNodeState  # noqa: F401
