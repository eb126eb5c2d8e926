"""Constants shared with the reference (gear/config.py:3)."""
KEY_T_RANGE = 2**31 - 1
