"""CPU oracle for the INT8 quantized-operator path.  Test infrastructure only:
imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg."""
from .qref import *  # noqa: F401,F403
