"""CPU oracle (test infrastructure only): ctypes bindings over libfv_oracle.so.

Only tests/, the smoke check and bench.py's cpu_baseline leg may import this
package. It is the parity checker and the timed CPU baseline, never the
product path.
"""
from .binding import *  # noqa: F401,F403
from .kv_cache import *  # noqa: F401,F403,E402
