"""Constants kept for source compatibility with upstream ``stickbreaking_attention/utils.py``."""
import math

PACKAGE_NAME = "stickbreaking_attention"
log2 = math.log(2)
inv_log2 = 1 / log2
