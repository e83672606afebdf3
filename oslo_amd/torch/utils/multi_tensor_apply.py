"""``MultiTensorApply`` of ``oslo/torch/utils/multi_tensor_apply/multi_tensor_apply.py``:
forwards a chunk size and a no-op flag to a multi-tensor kernel."""


class MultiTensorApply(object):
    def __init__(self, chunk_size):
        self.chunk_size = chunk_size

    def __call__(self, op, noop_flag_buffer, tensor_lists, *args):
        return op(self.chunk_size, noop_flag_buffer, tensor_lists, *args)


# the instance the optimizers share (oslo/torch/utils/multi_tensor_apply/__init__.py:3)
multi_tensor_applier = MultiTensorApply(2048 * 32)
