"""Architectures: each module registers one `config.registry.Architecture`."""
