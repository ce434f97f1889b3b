"""lucciola_amd: a small, whole inference engine for the Qwen3 dense decoder on one MI355X.

The Python entry points follow the reference's names (include/async_engine.h,
include/scheduler.h, include/sequence.h):

    from lucciola_amd import AsyncEngine
    engine = AsyncEngine(model_path, max_blocks=0, block_size=16)
    engine.generate_async(prompt_token_ids, max_new_tokens, callback)   # callback(token, finished)
    engine.stop()

and, stepped by the caller: ``LLMEngine`` (``add_request`` / ``step`` / ``generate``),
``Scheduler`` (``add_request`` / ``step`` / ``has_unfinished_requests`` / ``free_sequence``),
``Sequence``, ``SamplingParams``, ``EngineConfig``.  Requests carry token ids; where the model
folder holds a ``vocab.json``, ``generate_async`` also takes a string as the reference does
(``VocabTokenizer``, ``ChatFormat``) and calls back with text.
"""
__version__ = "0.1.0"

_LAZY = {
    "AsyncEngine": ("lucciola_amd.engine.async_engine", "AsyncEngine"),
    "LLMEngine": ("lucciola_amd.engine.llm_engine", "LLMEngine"),
    "ModelRunner": ("lucciola_amd.engine.runner", "ModelRunner"),
    "StepEntry": ("lucciola_amd.engine.batch", "StepEntry"),
    "Scheduler": ("lucciola_amd.engine.scheduler", "Scheduler"),
    "Sequence": ("lucciola_amd.engine.sequence", "Sequence"),
    "SequenceStatus": ("lucciola_amd.engine.sequence", "SequenceStatus"),
    "SamplingParams": ("lucciola_amd.sampling.sampler", "SamplingParams"),
    "EngineConfig": ("lucciola_amd.config.engine_config", "EngineConfig"),
    "Qwen3Config": ("lucciola_amd.config.model_config", "Qwen3Config"),
    "load_model": ("lucciola_amd.engine.loading", "load_model"),
    "random_model": ("lucciola_amd.engine.loading", "random_model"),
    "VocabTokenizer": ("lucciola_amd.text.vocab_tokenizer", "VocabTokenizer"),
    "ChatFormat": ("lucciola_amd.text.vocab_tokenizer", "ChatFormat"),
    "write_model_folder": ("lucciola_amd.weights.random_init", "write_model_folder"),
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        module, attr = _LAZY[name]
        return getattr(importlib.import_module(module), attr)
    raise AttributeError(f"module 'lucciola_amd' has no attribute '{name}'")


__all__ = sorted(_LAZY)
