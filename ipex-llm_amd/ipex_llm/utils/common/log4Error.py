"""Error convention of the low-bit linear path: log a banner, raise RuntimeError.

Mirrors python/llm/src/ipex_llm/utils/common/log4Error.py:22-41.
"""
import logging

logger = logging.getLogger(__name__)


def outputUserMessage(errMsg, fixMsg=None):
    logger.error("\n\n" + "*" * 28 + "Usage Error" + "*" * 24 + "\n" + errMsg)
    if fixMsg:
        logger.error("\n\n" + "*" * 26 + "How to fix" + "*" * 23 + "\n" + fixMsg)


def invalidInputError(condition, errMsg, fixMsg=None):
    if not condition:
        outputUserMessage(errMsg, fixMsg)
        raise RuntimeError(errMsg)


def invalidOperationError(condition, errMsg, fixMsg=None, cause=None):
    if not condition:
        outputUserMessage(errMsg, fixMsg)
        if cause:
            raise cause
        raise RuntimeError(errMsg)
