"""Instruction wire format of the decode megakernel.

An instruction is a flat run of int32 words: the opcode first, then every
dataclass field in declaration order.  Scalars take one word, sequences are
length-prefixed (``len, *items``) and ``None`` becomes a single 0.  The run is
zero-padded to ``INTS_PER_INSTRUCTION`` words when a queue is tensorized.

Wire-compatible with the reference encoder
(`qimeng_megakernel/models/instruction.py:15-35`), so instruction tensors
built by either side decode identically on the device.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, ClassVar, Iterable, Mapping, Sequence

INTS_PER_INSTRUCTION = 32


def _encode_field(value: Any) -> list[int]:
    # bool is an int subclass and is written as 0/1, like every other scalar.
    if isinstance(value, int):
        return [int(value)]
    if isinstance(value, (list, tuple)):
        return [len(value), *(int(v) for v in value)]
    if value is None:
        return [0]
    raise ValueError(f"instruction field of type {type(value).__name__} has no wire encoding")


@dataclasses.dataclass
class Instruction:
    """Base class: subclasses are dataclasses whose fields are the operand words."""

    OPCODE: ClassVar[int] = -1
    PREV_OPCODES: ClassVar[tuple[int, ...]] = ()

    @classmethod
    def opcode(cls) -> int:
        if cls.OPCODE < 0:
            raise NotImplementedError(f"{cls.__name__} declares no opcode")
        return cls.OPCODE

    @classmethod
    def prev_opcode(cls) -> tuple[int, ...]:
        return cls.PREV_OPCODES

    def serialize(self) -> list[int]:
        words = [self.opcode()]
        for f in dataclasses.fields(self):
            words.extend(_encode_field(getattr(self, f.name)))
        return words

    def padded(self, width: int = INTS_PER_INSTRUCTION) -> list[int]:
        words = self.serialize()
        if len(words) > width:
            raise ValueError(
                f"{type(self).__name__} needs {len(words)} words, the slot holds {width}"
            )
        return words + [0] * (width - len(words))


def run_pyvm_sequence(
    globs: Any,
    instructions: Iterable[Instruction],
    handler_map: Mapping[type, Callable[[Any, Instruction], None]],
) -> None:
    """Execute instructions one after another with the handler registered for each type.

    Same contract as the reference executor
    (`qimeng_megakernel/models/instruction.py:38-48`): a missing handler is a KeyError.
    """
    for ins in instructions:
        try:
            handler = handler_map[type(ins)]
        except KeyError:
            raise KeyError(f"Missing solver for instruction: {type(ins).__name__}") from None
        handler(globs, ins)


def decode_words(words: Sequence[int], classes: Mapping[int, type]) -> Instruction:
    """Inverse of ``serialize`` for one padded slot (used by tests and debugging tools)."""
    opcode = int(words[0])
    cls = classes[opcode]
    cursor = 1
    kwargs: dict[str, Any] = {}
    for f in dataclasses.fields(cls):
        is_seq = "list" in str(f.type) or "tuple" in str(f.type)
        if is_seq:
            n = int(words[cursor])
            kwargs[f.name] = [int(w) for w in words[cursor + 1 : cursor + 1 + n]]
            cursor += 1 + n
        else:
            raw = int(words[cursor])
            kwargs[f.name] = bool(raw) if "bool" in str(f.type) else raw
            cursor += 1
    return cls(**kwargs)
