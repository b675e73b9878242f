"""Parallel gradient accumulation into shared parameter slots (GPU)."""
from . import _lib

GLOBAL_ATOMICS = 0
LDS = 1
WAVE_LDS = 2
WAVE_LDS_SHALLOW = 3
LDS_LEAVES = 4
GLOBAL_LEAVES = 5
LDS_F32 = 6
AUTO = 7

STRATEGIES = {
    "global_atomics": GLOBAL_ATOMICS,
    "lds": LDS,
    "wave_lds": WAVE_LDS,
    "wave_lds_shallow": WAVE_LDS_SHALLOW,
    "lds_f32": LDS_F32,
    "auto": AUTO,
    "lds_leaves": LDS_LEAVES,
    "global_leaves": GLOBAL_LEAVES,
}

WIDTH = 6  # gradients per slot
BYTES_PER_THREAD = 28  # six fp32 inputs + one int32 slot index
DEFAULT = AUTO


def accumulate_chain_gradients(inputs, slot, grads, strategy=DEFAULT, stream=None):
    """Adds every thread's six chain gradients into row slot[i] of `grads`.

    inputs: six float32 CUDA tensors of length n; slot: int32 CUDA tensor of length n;
    grads:  float32 CUDA tensor of shape (num_slots, 6), contiguous, pre-initialised
            (the call only adds).  Returns `grads`.
    """
    import torch

    lib = _lib.load()
    if isinstance(strategy, str):
        strategy = STRATEGIES[strategy]
    n = slot.numel()
    if len(inputs) != 6:
        raise ValueError("expected 6 input arrays, got %d" % len(inputs))
    for t in inputs:
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n):
            raise ValueError("inputs must be contiguous float32 CUDA tensors of the slot array's length")
    if not (slot.is_cuda and slot.dtype == torch.int32 and slot.is_contiguous()):
        raise ValueError("slot must be a contiguous int32 CUDA tensor")
    if not (grads.is_cuda and grads.dtype == torch.float32 and grads.is_contiguous() and grads.dim() == 2 and grads.shape[1] == WIDTH):
        raise ValueError("grads must be a contiguous float32 CUDA tensor of shape (num_slots, 6)")
    s = stream if stream is not None else torch.cuda.current_stream(slot.device)
    with torch.cuda.device(slot.device):
        st = lib.xad_accumulate_chain_gradients_f32(
            int(strategy), n, *[t.data_ptr() for t in inputs], slot.data_ptr(), grads.data_ptr(), grads.shape[0], s.cuda_stream
        )
    _lib.check(st, "xad_accumulate_chain_gradients_f32")
    return grads


def zipf_(slot, seed, stream_id, num_slots, exponent=1.1):
    """Fills int32 CUDA tensor `slot` with Zipf(exponent) indices in [0, num_slots)."""
    import torch

    assert slot.is_cuda and slot.dtype == torch.int32 and slot.is_contiguous()
    with torch.cuda.device(slot.device):
        st = _lib.load().xad_rng_zipf_i32(slot.data_ptr(), slot.numel(), seed, stream_id, num_slots, exponent,
                                          torch.cuda.current_stream(slot.device).cuda_stream)
    _lib.check(st, "xad_rng_zipf_i32")
    return slot
