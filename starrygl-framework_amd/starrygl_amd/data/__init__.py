from .pipeline import MiniBatch, MiniBatchPipeline, MiniBatchPipelinePool  # noqa: F401
