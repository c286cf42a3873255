"""Engine-side accounting of sequence slots and 2 MiB chunks."""
from .chunk_manager import AllocStatus, ChunkSpaceManager, SequenceChunks  # noqa: F401
