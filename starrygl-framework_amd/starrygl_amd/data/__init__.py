from .loader import EventBatchLoader  # noqa: F401
from .pipeline import (GroupedMiniBatch, MiniBatch, MiniBatchGroup, MiniBatchGroupPipeline,  # noqa: F401
                       MiniBatchGroupPool, MiniBatchPipeline, MiniBatchPipelinePool)
