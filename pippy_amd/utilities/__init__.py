"""Utilities around the pipeline hot path (checkpoint I/O)."""
