"""Configuration errors.

A configuration problem is reported once, with every offending field, so that
a user fixes a config.json in one pass.  The reference collects all invalid
runtime fields into one error the same way
(v3/crates/rvllm-core/src/config/builder.rs:61-133).
"""

from __future__ import annotations


class ConfigError(ValueError):
    """One error that lists every problem found in a configuration."""

    def __init__(self, source: str, problems: list[str]):
        self.source = source
        self.problems = list(problems)
        lines = [f"{source}: {len(self.problems)} problem(s)"]
        lines += [f"  - {p}" for p in self.problems]
        super().__init__("\n".join(lines))


class UnknownArchitectureError(ConfigError):
    """config.json names an architecture that nobody registered."""
