"""Sizes beyond which the kernels refuse to run.  They are properties of the kernels, not of any model: a configuration
that exceeds one is refused with an error naming the limit when the model is built, a step when it is submitted."""

MAX_HEAD_DIM = 256        # attention keeps a head's accumulators in a wave's registers
MAX_EXPERTS = 1024        # the routing kernels keep a row's keys in one workgroup's LDS
MAX_TOP_K = 256           # picks per token the routing and combine kernels take
MAX_STEP_ROWS = 65535     # token rows of one step: several kernels put the rows into a grid's second dimension
