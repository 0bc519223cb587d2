"""MI355X-native LFM2 continuous-batching decode/prefill engine (drop-in for climbing-gym's native path).

Reference module -> module of this package:
  inference/lfm25_engine.py        -> engine.py, weights.py, cache.py, config.py
  inference/lfm25_cuda.py          -> decoder.py
  inference/lfm25_cuda_kernels.py, lfm25_fp8.py, lfm25_fp8_kv.py, lfm25_batching.py, lfm25_sampling.py -> ops.py
  inference/lfm25_session.py       -> session.py
  inference/text_stops.py          -> text_stops.py
  inference/lfm25_async_engine.py  -> async_engine.py;  inference/config.py, types.py -> inference_config.py, types.py
  inference/benchmark.py           -> benchmark.py;     rollout/{runner,config,contracts,coordinator}.py -> rollout.py
"""
from .config import LFM2Config, LFM25SamplingConfig

__all__ = ["LFM2Config", "LFM25SamplingConfig", "LFM25Engine", "LFM25PackedWeights", "LFM25HybridCache",
           "LFM25PrefixBatch", "LFM25DecodeBatch", "LFM25StepOutput", "LFM25GenerationOutput", "LFM25HIPDecoder",
           "LFM25CUDADecoder", "LFM25GenerationSession", "LFM25ContinuationHandle", "LFM25SessionResult",
           "flatten_token_batches", "LFM25AsyncInferenceEngine", "SamplingConfig", "InferenceEngineConfig",
           "GenerationOutput", "GenerationResult", "RolloutRunner", "RolloutRunnerConfig", "RolloutConfig",
           "RolloutCoordinator", "RolloutCoordinatorConfig", "DirectHarness"]

_LAZY = {
    "LFM25Engine": "engine", "LFM25PrefixBatch": "engine", "LFM25DecodeBatch": "engine", "LFM25StepOutput": "engine",
    "LFM25GenerationOutput": "engine", "flatten_token_batches": "engine", "LFM25PackedWeights": "weights",
    "LFM25HybridCache": "cache", "LFM25HIPDecoder": "decoder", "LFM25CUDADecoder": "decoder",
    "LFM25GenerationSession": "session", "LFM25ContinuationHandle": "session", "LFM25SessionResult": "session",
    "LFM25AsyncInferenceEngine": "async_engine", "SamplingConfig": "inference_config",
    "InferenceEngineConfig": "inference_config", "GenerationOutput": "types", "GenerationResult": "types",
    "RolloutRunner": "rollout", "RolloutRunnerConfig": "rollout", "RolloutConfig": "rollout",
    "RolloutCoordinator": "rollout", "RolloutCoordinatorConfig": "rollout", "DirectHarness": "rollout",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module(f".{_LAZY[name]}", __name__), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
