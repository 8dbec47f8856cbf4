"""ipex_llm.transformers: AutoModel* shells and the low-bit linear modules."""

_LAZY = {"AutoModelForCausalLM", "AutoModel", "AutoModelForSeq2SeqLM", "AutoModelForSequenceClassification"}


def __getattr__(name):
    # importing Hugging Face transformers takes seconds: only on first use
    if name in _LAZY:
        from . import model
        return getattr(model, name)
    raise AttributeError(name)
