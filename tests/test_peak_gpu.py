"""The measurement kernels of the library (fa_mfma_peak, fa_hbm_read_peak, fa_lds_read_peak) launch, finish and report what
they did; sizes are small, the rates are bench.py's business."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _lib():
    from flash_attn import _native as nat
    lib = nat.lib
    lib.fa_hbm_read_peak.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p]
    lib.fa_hbm_read_peak.restype = ctypes.c_int
    lib.fa_lds_read_peak.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64),
                                     ctypes.c_void_p, ctypes.c_void_p]
    lib.fa_lds_read_peak.restype = ctypes.c_int
    lib.fa_mfma_peak.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p]
    lib.fa_mfma_peak.restype = ctypes.c_int
    return lib


@pytest.mark.parametrize("nbytes", [16, 4096 * 16 + 16, 64 << 20, (64 << 20) + 16 * 12345])
@pytest.mark.parametrize("nontemporal", [0, 1])
def test_hbm_read_peak_reads_any_multiple_of_16_bytes(nbytes, nontemporal):
    print("hbm read peak", nbytes, nontemporal, flush=True)
    lib = _lib()
    src = torch.full((nbytes,), 7, dtype=torch.uint8, device=DEV)
    guard = torch.full((4096,), 9, dtype=torch.uint8, device=DEV)
    sink = torch.zeros(1, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.fa_hbm_read_peak(src.data_ptr(), nbytes, nontemporal, sink.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert int(sink.item()) == 0 and bool((src == 7).all()) and bool((guard == 9).all())     # nothing written
    # argument errors: no launch
    assert lib.fa_hbm_read_peak(None, nbytes, nontemporal, sink.data_ptr(), stream) != 0
    assert lib.fa_hbm_read_peak(src.data_ptr() + 8, 16, nontemporal, sink.data_ptr(), stream) != 0
    assert lib.fa_hbm_read_peak(src.data_ptr(), 8, nontemporal, sink.data_ptr(), stream) != 0


@pytest.mark.parametrize("random_operands", [0, 1])
def test_mfma_peak_counts_its_operations(random_operands):
    print("mfma peak", random_operands, flush=True)
    lib = _lib()
    sink = torch.zeros(1, dtype=torch.float32, device=DEV)
    flops = ctypes.c_int64(0)
    assert lib.fa_mfma_peak(sink.data_ptr(), 10, random_operands, ctypes.byref(flops), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert flops.value == 1024 * 4 * 10 * 16 * 2 * 32 * 32 * 16 and float(sink.item()) == 0.0
    assert lib.fa_mfma_peak(sink.data_ptr(), 0, random_operands, ctypes.byref(flops), None) != 0
    # the other instruction shape: twice the instructions, the same count of operations
    lib.fa_mfma_peak_shape.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p]
    lib.fa_mfma_peak_shape.restype = ctypes.c_int
    flops2 = ctypes.c_int64(0)
    assert lib.fa_mfma_peak_shape(sink.data_ptr(), 10, random_operands, 1, ctypes.byref(flops2), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert flops2.value == flops.value and float(sink.item()) == 0.0
    assert lib.fa_mfma_peak_shape(sink.data_ptr(), 10, random_operands, 2, ctypes.byref(flops2), None) != 0


@pytest.mark.parametrize("waves", [1, 4, 8, 16])
def test_lds_read_peak_reports_cycles_and_bytes(waves):
    print("lds read peak", waves, flush=True)
    lib = _lib()
    wgs = 64
    cycles = torch.zeros(wgs + 8, dtype=torch.int64, device=DEV)
    sink = torch.zeros(1, dtype=torch.int32, device=DEV)
    nbytes = ctypes.c_int64(0)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.fa_lds_read_peak(cycles.data_ptr(), wgs, waves, 100, ctypes.byref(nbytes), sink.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert nbytes.value == waves * 100 * 16 * 1024
    c = cycles.cpu()
    assert bool((c[:wgs] > 0).all()) and bool((c[wgs:] == 0).all()) and int(sink.item()) == 0
    rate = nbytes.value / c[:wgs].double().mean().item()
    assert 8.0 < rate < 1024.0, rate          # bytes per clock of one CU: a sane order of magnitude
    for bad in ((0, waves), (wgs, 0), (wgs, 17)):
        assert lib.fa_lds_read_peak(cycles.data_ptr(), bad[0], bad[1], 100, ctypes.byref(nbytes), sink.data_ptr(), stream) != 0
