"""Builds the oracle's native parts (test infrastructure)."""


def build_all(force=True, verbose=False):
    pass
