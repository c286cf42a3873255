"""Engine-side accounting of sequence slots and 2 MiB chunks, and the step scheduler over it."""
from .chunk_manager import AllocStatus, ChunkSpaceManager, SequenceChunks  # noqa: F401
from .scheduler import PreemptionMode, Request, SchedulerOutputs, SeqStatus, StepScheduler  # noqa: F401
