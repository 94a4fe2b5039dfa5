from atomserve_amd.engine.batch import Row, StepBatch, slot_of
from atomserve_amd.engine.scheduler import Scheduler, SchedulerOutput
from atomserve_amd.engine.sequence import (
    NON_THINKING_PARAMS,
    THINKING_PARAMS,
    SamplingParams,
    Sequence,
    SequenceStatus,
    StepResult,
)

__all__ = ["NON_THINKING_PARAMS", "Row", "SamplingParams", "Scheduler", "SchedulerOutput", "Sequence",
           "SequenceStatus", "StepBatch", "StepResult", "THINKING_PARAMS", "slot_of"]  # fmt: skip
