"""Architectures: each module registers one ``config.json`` architecture name."""
