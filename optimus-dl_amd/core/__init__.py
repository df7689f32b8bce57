"""Minimal core: the registry and the dtype tables that the FP8 path needs."""
