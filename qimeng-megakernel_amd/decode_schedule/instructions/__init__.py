"""Instruction definitions and the host-side scheduler of the MI355X decode route."""
from . import instruction_defs, scheduler
from .instruction_defs import *  # noqa: F401,F403
from .scheduler import (  # noqa: F401
    build,
    build_instruction_list,
    build_instruction_queues,
    tensorize_instructions,
)
