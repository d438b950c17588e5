"""Instruction set and scheduler of the batch route."""
