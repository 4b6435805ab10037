"""User-level TorchScript programs of the benchmark configurations (imperative
tensor programs with in-place writes, as a user of functs.jit writes them)."""
from .programs import (PROGRAMS, attention_steps, delta2bbox, get_started, lstm, ssd_postproc, yolov3_batched,  # noqa: F401
                       yolov3_head, yolov3_postproc)
