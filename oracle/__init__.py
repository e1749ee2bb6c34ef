"""CPU oracle package - TEST INFRASTRUCTURE ONLY (see spattn_oracle.py).

Nothing under fgattn_tk_cuda_amd/ imports this package.
"""
