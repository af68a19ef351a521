from .triangle_multiplication import (TriangleMultiplication, TriangleMultiplicationFunction,  # noqa: F401
                                      channels_first_to_last, channels_last_to_first, trimul_pack_backward,
                                      trimul_pack_forward)
