"""Logger factory with the ``[MLF <time> <level> Step=<s> Rank=<r> <name>:<line>] <msg>`` line format.

Format and the ``MLFLASHPOINT_LOG_LEVEL`` switch follow the reference
(src/ml_flashpoint/core/mlf_logging.py:64-111).  The default level here is WARNING rather than DEBUG so that the
per-buffer INFO lines do not sit on the save path unless asked for.
"""

import logging
import multiprocessing
import os
import sys

_TRAINING_STEP = multiprocessing.Value("i", -1)
_RANK = -1


def update_training_step(new_val: int) -> None:
    with _TRAINING_STEP.get_lock():
        _TRAINING_STEP.value = new_val


def get_current_step() -> int:
    return _TRAINING_STEP.value


def setup_worker_logging(rank: int, step: int) -> None:
    global _RANK
    _RANK = rank
    update_training_step(step)


class TrainingContextFormatter(logging.Formatter):
    def format(self, record):
        record.curr_step = get_current_step()
        rank = _RANK
        if rank < 0:
            try:
                import torch.distributed as dist

                if dist.is_available() and dist.is_initialized():
                    rank = dist.get_rank()
            except Exception:
                pass
        record.rank = rank
        return super().format(record)


def get_logger(name: str, stream=sys.stderr) -> logging.Logger:
    logger = logging.getLogger(name)
    if not logger.handlers:
        handler = logging.StreamHandler(stream=stream)
        handler.setFormatter(
            TrainingContextFormatter(
                "[MLF %(asctime)s %(levelname)s Step=%(curr_step)s Rank=%(rank)s %(name)s:%(lineno)d] %(message)s"
            )
        )
        logger.addHandler(handler)
        level = os.environ.get("MLFLASHPOINT_LOG_LEVEL", "WARNING").upper()
        logger.setLevel(logging._nameToLevel.get(level, logging.WARNING))
    logger.propagate = False
    return logger
