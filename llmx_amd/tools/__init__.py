"""Command-line tools built on the engine."""
