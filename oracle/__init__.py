"""CPU oracle for the jsgrad Llama-3 inference path -- test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package.  The product (denograd_amd) never does.
"""
from .oracle import *  # noqa: F401,F403
