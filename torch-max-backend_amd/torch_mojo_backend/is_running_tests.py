"""Test-mode switch (reference: torch_mojo_backend/is_running_tests.py:3). When set, every
registry entry and eager registration counts its calls so tests can prove which
implementation ran."""

import os

IS_RUNNING_TESTS = os.environ.get("TORCH_MOJO_BACKEND_TESTING", "0") == "1"
