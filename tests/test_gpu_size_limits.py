"""The kernels address their operands with 32-bit offsets: an operand of 2^31 elements or
more (a grid beyond the launch limits, an attention shape without a kernel) is refused with
PET_HIP_ERR_UNSUPPORTED before anything is launched. The reference maps an unsupported shape
to perf() = INFINITY (include/operator.h:176-252); here the host layer does that with the
status. The pointers are small real buffers: a call that got past its checks would be
caught by the shapes' own size."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

UNSUPPORTED = 2


@pytest.fixture(scope="module")
def buf():
    from pet_amd import abi
    abi.init(0)
    t = torch.zeros(64, device="cuda")
    return abi, ctypes.c_void_p(t.data_ptr()), t


def ints(*v):
    return (ctypes.c_int * len(v))(*v)


def refused(abi, name, *args):
    with pytest.raises(abi.PetHipError) as e:
        abi.call(name, *args)
    assert e.value.status == UNSUPPORTED, str(e.value)


def test_convolutions_refuse_operands_of_2_31_elements(buf):
    abi, p, _ = buf
    # input 1 x 65536 x 256 x 256 = 2^32 elements
    refused(abi, "pet_hip_conv2d_f32", p, p, None, p, 1, 65536, 256, 256, 1, 1, 1, 0, 0, 1, 1, 1,
            1, 1, 0, None)
    # output 1 x 32768 x 256 x 256 = 2^31 elements
    refused(abi, "pet_hip_conv2d_f32", p, p, None, p, 1, 1, 256, 256, 32768, 1, 1, 0, 0, 1, 1, 1,
            1, 1, 0, None)
    # 3-D: input 1 x 8 x 1024 x 1024 x 256 = 2^31 elements
    refused(abi, "pet_hip_conv3d_f32", p, p, None, p, 1, 8, 1024, 1024, 256, 1, 1, 1, 1, 0, 0, 0,
            1, 1, 1, 1, 1, 1, 1, 0, None)
    # transposed: input 1 x 65536 x 32768 x 1
    refused(abi, "pet_hip_conv_trans_f32", p, p, None, p, 1, 65536, 32768, 1, 1, 1, 1, 0, 0, 1,
            1, 1, 1, 0, 0, 0, None)


def test_matmuls_refuse_operands_of_2_31_elements(buf):
    abi, p, _ = buf
    refused(abi, "pet_hip_bmm_f32", 0, 0, 1, 65536, 1, 32768, p, p, p, None, 0, None)   # A
    refused(abi, "pet_hip_bmm_f32", 0, 0, 1, 1, 65536, 32768, p, p, p, None, 0, None)   # B
    refused(abi, "pet_hip_bmm_f32", 0, 0, 1, 65536, 32768, 1, p, p, p, None, 0, None)   # C
    refused(abi, "pet_hip_bmm_f32", 1, 1, 70000, 2, 2, 2, p, p, p, None, 0, None)       # grid z
    refused(abi, "pet_hip_g2bmm_f32", p, p, p, 1, 1 << 20, 2048, 1, 1, None)
    refused(abi, "pet_hip_g2bmm_f32", p, p, p, 1, 1 << 20, 32, 1024, 1, None)           # the band
    refused(abi, "pet_hip_gbmml_f32", p, p, p, 1, 1 << 20, 2048, 1, 1, None)
    refused(abi, "pet_hip_g2bmm_f32", p, p, p, 40000, 4, 4, 1, 2, None)                 # grid z


def test_layout_operators_refuse_tensors_of_2_31_elements(buf):
    abi, p, _ = buf
    refused(abi, "pet_hip_transpose", p, p, ints(65536, 32768), ints(1, 0), 2, None)
    refused(abi, "pet_hip_pad", p, p, ints(65536, 32767), ints(0, 0), ints(0, 1), 2, None)


def test_attention_refuses_shapes_without_a_kernel(buf):
    abi, p, _ = buf

    def attn(seq, dh, heads=2, batch=1):
        w = heads * dh
        return ("pet_hip_attention_f32", p, p, p, p, batch, heads, seq, dh, w, w, w, w,
                seq * w, seq * w, seq * w, seq * w, 1.0, None, None)
    refused(abi, *attn(513, 64))
    refused(abi, *attn(64, 48))
    refused(abi, *attn(64, 64, batch=70000))
