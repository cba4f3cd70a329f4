

def load_runner(path: str, **kw):
    """The runner class follows the model: a folder with config.json + model.safetensors is a layer-list model
    (`StackRunner`; accepts dtype=, kv_tokens=), a GGUF file a `Runner` (accepts ext_rows=, tp_*=). Both serve the
    same interface to the scheduler, the server and the command line."""
    from ..models.config import is_stack_model
    if is_stack_model(path):
        from .stack_runner import StackRunner
        kw.pop("ext_rows", None)
        return StackRunner(path, **kw)
    from .runner import Runner
    kw.pop("dtype", None)
    return Runner(path, **kw)
