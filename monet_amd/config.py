"""Process-wide settings read by the operator library.

`budget` is the memory budget in GB that autotuning conv ops must stay under
(the role of the reference's top-level config.py:1); 0 means "no limit".
"""
budget = 0
