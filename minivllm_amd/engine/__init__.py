from .block_manager import Block, BlockManager  # noqa: F401
from .scheduler import Scheduler  # noqa: F401
from .sequence import Sequence, SequenceStatus  # noqa: F401
