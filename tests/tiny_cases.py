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


class ViewNet:
    """A network that needs strided views: an NCHW qsi8 image is read through a DIMSHUFFLE view
    as [N, C/4, H, W, 4] and made dense by Relayout (how an NCHW model enters NCHW44 kernels),
    max- and average-pooled, the two results joined by Concat along the channel blocks, and the
    last two blocks taken out again through a SUBTENSOR view + Relayout."""
    N, C, H, W = 2, 8, 6, 6
    SCALE = 0.05

    def __init__(self):
        from cases import PoolCase
        from megcc_amd import abi
        self.pool_max = PoolCase(abi.FMT_NCHW44, abi.POOL_MAX, self.N, self.C, self.H, self.W,
                                 2, 2, 0, scale=self.SCALE)
        self.pool_avg = PoolCase(abi.FMT_NCHW44, abi.POOL_AVERAGE, self.N, self.C, self.H, self.W,
                                 2, 2, 0, scale=self.SCALE)

    def build(self, m):
        """m: runtime.Model or tiny.ModelBuilder"""
        from megcc_amd import abi
        n, c, h, w = self.N, self.C, self.H, self.W
        q = lambda name, shape: m.tensor(name, shape, abi.QINT8, self.SCALE)
        ids = {}
        ids["image"] = q("image", (n, c, h, w))
        m.mark_input(ids["image"])
        blocked = (n, c // 4, h, w, 4)
        v = m.view("image.as_nchw4", ids["image"], blocked, (c * h * w, 4 * h * w, w, 1, h * w))
        ids["x4"] = q("x4", blocked)
        m.opr("GI_kernel_relayout_qsi8", [v], [ids["x4"]])
        half = (n, c // 4, h // 2, w // 2, 4)
        ids["max"], ids["avg"] = q("max", half), q("avg", half)
        m.opr(self.pool_max.symbol(), [ids["x4"]], [ids["max"]])
        m.opr(self.pool_avg.symbol(), [ids["x4"]], [ids["avg"]])
        both = (n, c // 2, h // 2, w // 2, 4)
        ids["cat"] = q("cat", both)
        m.opr("kernel_concat_byte_1_axis_1", [ids["max"], ids["avg"]], [ids["cat"]])
        plane = (h // 2) * (w // 2) * 4
        tail = m.view("cat.tail", ids["cat"], half,
                      (c // 2 * plane, plane, (w // 2) * 4, 4, 1), offset=(c // 4) * plane)
        ids["out"] = q("out", half)
        m.opr("GI_kernel_relayout_qsi8", [tail], [ids["out"]])
        m.mark_output(ids["cat"])
        m.mark_output(ids["out"])
        m.finalize()
        return ids

    def draw_input(self, seed):
        return np.random.default_rng(seed).integers(
            -128, 128, (self.N, self.C, self.H, self.W)).astype(np.int8)

    def run_oracle(self, image):
        """-> (cat, out), from the pooling port and numpy's own transpose / concatenate"""
        from oracle import port
        n, c, h, w = image.shape
        x4 = np.ascontiguousarray(image.reshape(n, c // 4, 4, h, w).transpose(0, 1, 3, 4, 2))
        a = self.pool_max.run_port({"src": x4})
        b = self.pool_avg.run_port({"src": x4})
        cat = np.concatenate([a, b], 1)
        return cat, np.ascontiguousarray(cat[:, c // 4:])
