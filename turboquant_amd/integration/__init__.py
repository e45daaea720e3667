"""Adapters that attach the compressed KV path to a serving engine."""
