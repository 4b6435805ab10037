"""User-level TorchScript programs of the benchmark configurations (imperative
tensor programs with in-place writes, as a user of functs.jit writes them)."""
from .programs import PROGRAMS, get_started, lstm, ssd_postproc, yolov3_batched, yolov3_postproc  # noqa: F401
