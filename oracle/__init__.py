"""CPU oracle for the Ferrox training hot path -- TEST INFRASTRUCTURE ONLY.

Importable only from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
The product package (ferrox_amd) never imports this module.
"""
from .binding import *  # noqa: F401,F403
from . import train  # noqa: F401
