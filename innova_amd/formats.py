"""Wire formats of .oil blocks, numbered as oil::Format (include/oil/types.h:19-35)."""
from enum import IntEnum

WIRE_BLOCK = 256  # weights per block on the wire (src/format_registry.cpp:17)


class Format(IntEnum):
    OIL1 = 0
    SPARK_Q0 = 1
    OIL2 = 2
    OIL4 = 3
    OIL8 = 4
    OIL16 = 5
    OIL32 = 6
    OIL1_GRP = 7
    SPARK_Q0_GRP = 8
    OIL2_GRP = 9
    OIL4_GRP = 10
    OIL8_GRP = 11
    OIL16_GRP = 12
    SPARK_SPARSE = 13
    SPARK_SPARSE_GRP = 14


_BPW = {Format.OIL1: 1.0, Format.SPARK_Q0: 1.5, Format.OIL2: 2.0, Format.OIL4: 4.0, Format.OIL8: 8.0,
        Format.OIL16: 16.0, Format.OIL32: 32.0, Format.OIL1_GRP: 1.0, Format.SPARK_Q0_GRP: 1.5,
        Format.OIL2_GRP: 2.5, Format.OIL4_GRP: 4.5, Format.OIL8_GRP: 8.5, Format.OIL16_GRP: 16.0,
        Format.SPARK_SPARSE: 2.0, Format.SPARK_SPARSE_GRP: 2.0}


def format_bpw(fmt) -> float:
    """Claimed bits per weight (include/oil/types.h:57-82)."""
    return _BPW.get(Format(int(fmt)), 0.0)


# stored payload bytes of one full 256-weight block
FULL_BLOCK_BYTES = {Format.OIL1: 16, Format.SPARK_Q0: 48, Format.OIL2: 64, Format.OIL4: 128,
                    Format.OIL8: 256, Format.OIL16: 512, Format.OIL32: 1024, Format.OIL1_GRP: 32,
                    Format.SPARK_Q0_GRP: 48, Format.OIL2_GRP: 80, Format.OIL4_GRP: 144,
                    Format.OIL8_GRP: 272, Format.OIL16_GRP: 512, Format.SPARK_SPARSE: 64,
                    Format.SPARK_SPARSE_GRP: 64}
