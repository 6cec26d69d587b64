"""Sizes the kernels take, in one place for the configuration classes and the parts that check them."""

MAX_HEAD_DIM = 256             # the widest attention head any kernel takes
MATRIX_CORE_HEAD_STEP = 16     # bfloat16 attention runs on the matrix cores for head sizes in these steps and on
                               # the plain kernel (float arithmetic, any size) for the rest
