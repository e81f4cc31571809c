from .engine import Engine
from .native import NativeEngine, NativeEngineError, load_plugin, native_support
from .scheduler import Scheduler
from .step import ModelRunner, StepEntry


def create_engine(model_dir, *, plugins=(), **options):
    """The engine for a model folder: the native engine when the library (with its plugins) has the model's
    architecture and every part kind it names, else the Python step function, for models made of parts that are
    registered in Python.  ``options`` are those of ``Engine`` / ``NativeEngine`` (dtype, num_pages, page_size,
    max_num_seqs, max_num_batched_tokens, enable_prefix_cache, max_model_len, graphs)."""
    for path in plugins:
        load_plugin(path)
    supported, _ = native_support(model_dir)
    return NativeEngine(model_dir, **options) if supported else Engine(model_dir, **options)


__all__ = ["Engine", "ModelRunner", "NativeEngine", "NativeEngineError", "Scheduler", "StepEntry", "create_engine", "load_plugin",
           "native_support"]
