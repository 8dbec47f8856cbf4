"""MI355X-native low-bit linear path behind the ipex-llm Python API."""


def __getattr__(name):
    # optimize_model pulls in torch / transformers machinery: import it on first use
    if name == "optimize_model":
        from .optimize import optimize_model
        return optimize_model
    raise AttributeError(name)
