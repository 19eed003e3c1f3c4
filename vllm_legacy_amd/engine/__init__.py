"""Serving engine: requests -> scheduler -> cache manager -> model runner -> sampler.

  LLMEngine.add_request / step / generate   engine/llm_engine.py
  Scheduler (continuous batching, prompts cut into portions under a token budget,
  preemption by recomputation)                engine/scheduler.py
  CacheManager (paged cache blocks + recurrent-state slots, both reused)
                                              engine/cache_manager.py
  ModelRunner (packs a step, runs the model, returns the logits asked for)
                                              engine/model_runner.py
  Sampler / SamplingParams                    engine/sampling.py
  trace replay (given steps instead of scheduled ones, logits to files)
                                              engine/trace_replay.py, bin/trace_run
  command line                                engine/cli.py
  the Llama decode stack behind the same protocol
                                              engine/llama_adapter.py
"""
from .cache_manager import CacheManager  # noqa: F401
from .llm_engine import EngineConfig, LLMEngine, RequestOutput  # noqa: F401
from .model_runner import ModelRunner  # noqa: F401
from .sampling import Sampler, SamplingParams  # noqa: F401
from .scheduler import Scheduler, Sequence  # noqa: F401
