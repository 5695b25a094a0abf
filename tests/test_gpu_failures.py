"""Failure handling on the GPU box: conditions forced from the host (an allocation the device cannot hold, a device
that does not exist, arguments a kernel would not survive) come back as the matching error class with a message,
and the context keeps working afterwards.  No kernel is made to fault: every refused call stops before a launch."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def still_works(ex, orc):
    x = np.arange(1, 65, dtype=np.float32).reshape(1, 64)
    g = np.ones(64, dtype=np.float32)
    assert np.allclose(ex.rmsnorm(x, g, 1e-5), orc.rmsnorm(x, g, 1e-5), rtol=1e-6)


def test_allocation_beyond_the_device_is_out_of_memory(ex, orc):
    from rustorch_amd import OutOfMemory
    with pytest.raises(OutOfMemory) as e:
        ex.buffer(1 << 46)                          # 64 TiB
    assert "hipMalloc" in str(e.value) or "memory" in str(e.value).lower()
    still_works(ex, orc)


def test_model_whose_cache_cannot_fit_is_out_of_memory(ex, orc):
    from rustorch_amd import llama, OutOfMemory
    with pytest.raises(OutOfMemory):
        llama.HipLlama(ex, n_layers=200_000, hidden=4096, n_heads=32, ffn=11008, vocab=32000, max_pos=16000)    # a 52 TB cache
    still_works(ex, orc)
    gm = llama.HipLlama(ex, n_layers=1, hidden=256, n_heads=2, ffn=512, vocab=100, max_pos=8)                # and a sane one still builds
    gm.close()


def test_device_that_does_not_exist(ex):
    from rustorch_amd import DeviceNotAvailable
    from rustorch_amd.executor import HipKernelExecutor
    with pytest.raises(DeviceNotAvailable):
        HipKernelExecutor(99)


def test_refused_arguments_leave_a_message_and_a_working_context(ex, orc):
    from rustorch_amd import synth, InvalidParameters, ShapeMismatch, UnsupportedOperation
    raw = synth.blocks(12, 1, 1, 8, 256)
    w = ex.upload_qweight(12, 8, 256, raw)
    with pytest.raises(ShapeMismatch):
        ex.qgemv(w, np.zeros(255, np.float32))
    with pytest.raises(InvalidParameters):
        ex.qgemv_dev(w, ex.to_device(np.zeros(256, np.float32)), ex.buffer(32), 0)      # batch 0
    with pytest.raises(UnsupportedOperation):
        ex.upload_qweight(15, 8, 256, np.zeros(8 * 292, np.uint8))                       # Q8_K: no kernel
    with pytest.raises(ShapeMismatch):
        ex.attn_decode(np.zeros(2 * 96, np.float32), np.zeros((4, 192), np.uint16), np.zeros((4, 192), np.uint16), 4, 2, 96)   # head_dim 96
    dx, dy = ex.to_device(np.zeros(8 * 256, np.float32)), ex.buffer(8 * 8 * 4)
    with pytest.raises(InvalidParameters):
        ex.qgemv_shared_x_dev([w] * 9, dx, [dy] * 9, 8)                                  # more than eight weights
    with pytest.raises(InvalidParameters):
        ex.qgemv_shared_x_dev([w], dx, [dy], 9)                                          # batch beyond eight
    with pytest.raises(InvalidParameters):
        ex.qgemv_shared_x_dev([w, w], dx, [dy], 8)                                       # one output for two weights
    still_works(ex, orc)
    y = ex.qgemv(w, np.ones(256, np.float32))
    assert np.isfinite(y).all()
