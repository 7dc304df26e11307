"""Errors of a step."""


class StepError(ValueError):
    """A step that cannot run: a dead slot, a token outside the vocabulary, no room."""
