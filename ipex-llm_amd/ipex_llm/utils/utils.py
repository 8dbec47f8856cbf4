"""Where the native library lives (python/llm/src/ipex_llm/utils/utils.py:22-41)."""
import pathlib


def get_shared_lib_info(lib_base_name: str):
    """Returns (directory, [candidate paths]) for lib<name>.so under ipex_llm/libs."""
    base = (pathlib.Path(__file__).parent.parent / "libs").resolve()
    return base, [base / f"lib{lib_base_name}.so"]
