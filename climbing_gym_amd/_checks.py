"""Argument and state checks in one line each: `reject(condition, text)` raises `kind(text)` when the condition holds.
The texts are the reference's (callers and tests match on them); the conditions are evaluated where the call stands,
so a check that reads the device synchronises there, as an `if` would."""
from __future__ import annotations


def reject(condition, text: str, kind=ValueError) -> None:
    if condition:
        raise kind(text)
