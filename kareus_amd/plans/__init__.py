"""Schedule files shipped with the package (the grammar of kareus/scheduler/parser.py:66-101,122-165,228-274)."""

import os


def plan_path(name: str) -> str:
    """Absolute path of a shipped plan file."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), name)
    if not os.path.exists(path):
        raise FileNotFoundError(path)
    return path
