from .loader import EventBatchLoader  # noqa: F401
from .pipeline import MiniBatch, MiniBatchPipeline, MiniBatchPipelinePool  # noqa: F401
