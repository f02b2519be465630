"""MI355X-native implementation of PiPPy's per-stage pipeline hot path.

Public names mirror ``pippy/__init__.py:26-43`` of the reference so that a script written against
``pippy`` runs against this package by changing the import.
"""
__version__ = "0.1.0"
