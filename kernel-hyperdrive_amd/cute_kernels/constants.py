"""Library-wide constants, rebuilt for gfx950 (wave64, 1024-lane workgroups, 16-byte vector access).

Replaces cute_kernels/constants.py:1-23; the Triton block-size lists and the torch->triton dtype map have
no meaning here and are gone.
"""

from .math import get_powers_of_2


LIBRARY_NAME = "cute"

WAVE_SIZE = 64
MAX_WORKGROUP_SIZE = 1024
# workgroup sizes the streaming kernels are tuned over: whole wavefronts only
COMMON_WORKGROUP_SIZES = get_powers_of_2(WAVE_SIZE, MAX_WORKGROUP_SIZE)

# names kept from the reference: elements of one 16-byte access
MAX_FP32_INSTRUCTION_WIDTH = 4
MAX_FP16_BF16_INSTRUCTION_WIDTH = 8
COMMON_VECTOR_INSTRUCTION_WIDTHS = get_powers_of_2(1, MAX_FP32_INSTRUCTION_WIDTH)

# longest row the RMSNorm kernels accept (the reference's MAX_TRITON_BLOCK_SIZE)
MAX_ROW_LENGTH = 65536

LDS_BYTES_PER_CU = 160 * 1024
