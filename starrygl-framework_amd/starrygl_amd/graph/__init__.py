from .graph import AsyncBlock, AsyncGraphBlob, Block, NegSamplingSet, pyGraph  # noqa: F401
