from .pipeline import MiniBatch, MiniBatchPipeline  # noqa: F401
