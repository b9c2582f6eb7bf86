"""Small `.tiny` model descriptions for the reader tests (no GPU needed to write or read them)."""
import numpy as np

from megcc_amd import tiny


def small_model():
    """Touches every table and field the loader reads: several dtypes, a weight without dtype
    parameters, explicit strides and formats, defaults present and absent, two device models,
    Opr / MemForward / DevMemAlloc / DevMemFree instructions, weight outputs."""
    r = np.random.default_rng(5)
    weights = [
        dict(name="w.q8", dtype=(tiny.QINT8, 0.0125), dims=[2, 1, 3, 3, 4, 4],
             data=r.integers(-127, 128, 288).astype(np.int8), use_count=2, checksum=77),
        dict(name="w.bias", dtype=(tiny.QINT32, 0.00025, 0), dims=[1, 2, 1, 1, 4],
             data=r.integers(-1000, 1000, 8).astype(np.int32)),
        dict(name="w.f16", dtype=(tiny.FLOAT32, None), dims=[3, 5], compressed=True,
             data=r.uniform(-2, 2, 15).astype(np.float16)),
        dict(name="w.u8", dtype=(tiny.QUINT8, 0.5, 128), dims=[6], format=tiny.FORMAT_OIHW,
             data=np.arange(6, dtype=np.uint8)),
    ]
    tensors = [
        dict(name="data", dtype=(tiny.FLOAT32, None), dims=[1, 4, 5, 5], use_count=1),
        dict(name="", dtype=(tiny.QINT8, 0.02), dims=[1, 1, 5, 5, 4], offset=0, use_count=1),
        dict(name="conv", dtype=(tiny.QINT8, 0.05), dims=[1, 2, 5, 5, 4], offset=128,
             stride=[200, 100, 20, 4, 1], format=tiny.FORMAT_NCHW4, use_count=2),
        dict(name="view", dtype=(tiny.QINT8, 0.05), dims=[1, 200], offset=128),
        dict(name="dyn", dtype=(tiny.INT32, None), dims=[7], dynamic=True),
    ]
    conv = "kernel_conv2d_3x3_NCHW44_DENSE_p1x1_s1x1_d1x1_qsi8qsi8qsi32qsi8_bias_RELU"
    instructions = [
        ("Opr", dict(name="cvt", type="kernel_typecvt_f32qsi8", inputs=[0], input_types=[0],
                     outputs=[1], kernel_id=0)),
        ("Opr", dict(name="conv", type=conv, inputs=[1, 0, 1], input_types=[0, 1, 1], outputs=[2],
                     workspace_size=4096, workspace_offset=512, init_id=3, kernel_id=1,
                     workspace_id=2, deduce_id=5)),
        ("MemForward", dict(input=2, output=3, offset=0, type=tiny.MEMFORWARD_RESHAPE)),
        ("DevMemAlloc", dict(tensor=4)),
        ("MemForward", dict(input=2, output=3, offset=40, type=tiny.MEMFORWARD_SUBTENSOR)),
        ("DevMemFree", dict(tensor=4)),
    ]
    first = dict(device=tiny.DEVICE_BARE_METAL, tensor_memory=4608, tensors=tensors,
                 instructions=instructions, inputs=[0], outputs=[3], weight_outputs=[1, 3],
                 weight_output_names=["bias_out", "u8_out"])
    second = dict(device=tiny.DEVICE_ARM64, tensor_memory=1 << 33, tensors=tensors[:2],
                  instructions=instructions[:1], inputs=[0], outputs=[1])
    return dict(name="small", model_id=0x1234567890abcdef, const_shape=False, weights=weights,
                device_models=[first, second])
