"""File logging of operator calls for enable(record=True).

Behaviour follows src/flag_gems/logging_utils.py:5-39 of the reference: a FileHandler on the
"flag_gems" logger at DEBUG level, optionally de-duplicated per call site.
"""
import logging
from pathlib import Path


class LogOncePerLocationFilter(logging.Filter):
    def __init__(self):
        super().__init__()
        self.seen = set()

    def filter(self, record):
        where = (record.pathname, record.lineno)
        if where in self.seen:
            return False
        self.seen.add(where)
        return True


def setup_flaggems_logging(path=None, record=True, once=False):
    if not record:
        return
    target = Path(path or Path.home() / ".flaggems/oplist.log")
    target.parent.mkdir(parents=True, exist_ok=True)
    handler = logging.FileHandler(target, mode="w")
    if once:
        handler.addFilter(LogOncePerLocationFilter())
    handler.setFormatter(logging.Formatter("[%(levelname)s] %(name)s: %(message)s"))
    logger = logging.getLogger("flag_gems")
    logger.setLevel(logging.DEBUG)
    if not any(isinstance(h, logging.FileHandler) for h in logger.handlers):
        logger.addHandler(handler)
    logger.propagate = False
