"""ctypes prototypes of the kernel-level C ABI (include/mchip/kernels.h).

Pointers are raw device addresses (ints); torch is only used by callers to own
device memory and streams.
"""
import ctypes

from .base import LIB, check_mc

c_void_p = ctypes.c_void_p
c_int = ctypes.c_int
c_float = ctypes.c_float

ACT_NONE, ACT_RELU, ACT_TANH, ACT_SIGMOID = 0, 1, 2, 3


class ConvGeom(ctypes.Structure):
    _fields_ = [(n, c_int) for n in (
        "channels_in", "height_in", "width_in", "channels_out", "kernel_h", "kernel_w",
        "stride_h", "stride_w", "pad_h", "pad_w", "dilation_h", "dilation_w", "group",
        "transposed")]


class Epilogue(ctypes.Structure):
    _fields_ = [("scale", c_void_p), ("shift", c_void_p), ("residual", c_void_p),
                ("activation", c_int), ("negative_slope", c_float)]


class ChannelOp(ctypes.Structure):
    _fields_ = [("sub", c_void_p), ("div", c_void_p), ("mul", c_void_p), ("add", c_void_p),
                ("activation", c_int), ("negative_slope", c_float)]


c_long = ctypes.c_long
LIB.mcChannelTransform.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int,
                                   ctypes.POINTER(ChannelOp), c_void_p]
LIB.mcBatchNormStored.argtypes = [c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_void_p,
                                  c_void_p]
LIB.mcBatchNormBatchStats.argtypes = [c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p,
                                      c_void_p]
LIB.mcFoldChannelOps.argtypes = [c_void_p, ctypes.POINTER(ChannelOp), c_int, c_int, c_void_p,
                                 c_void_p, c_void_p]
LIB.mcPoolingOutputShape.argtypes = [c_int] * 8 + [ctypes.POINTER(c_int), ctypes.POINTER(c_int)]
LIB.mcPooling.argtypes = [c_int, c_void_p, c_void_p] + [c_int] * 9 + [c_void_p]
LIB.mcEltwise.argtypes = [c_int, c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_float), c_long,
                          c_void_p, c_int, c_float, c_void_p]
LIB.mcSoftmax.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]
LIB.mcCopy2D.argtypes = [c_void_p, c_long, c_void_p, c_long, c_long, c_long, c_void_p]
LIB.mcConcat.argtypes = [ctypes.POINTER(c_void_p), ctypes.POINTER(ctypes.c_long), c_int, c_void_p, ctypes.c_long, c_void_p]
LIB.mcPermute.argtypes = [c_void_p, c_void_p, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                          c_void_p]
LIB.mcFill.argtypes = [c_void_p, c_long, c_float, c_void_p]
LIB.mcNormalize.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p,
                            c_void_p]
LIB.mcConvTimingCollect.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_long),
                                    ctypes.POINTER(ctypes.c_double)]
LIB.mcConvTimingCollectDetail.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_long),
                                          ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double),
                                          ctypes.POINTER(c_long)]

LIB.mcDetectionOutputWorkspaceSize.argtypes = [c_int, c_int, c_int, c_int, c_int,
                                               ctypes.POINTER(ctypes.c_size_t)]
LIB.mcDetectionOutputMaxRows.argtypes = [c_int] * 5
LIB.mcDetectionOutputSplit.argtypes = [c_int]
LIB.mcDetectionOutput.argtypes = [c_void_p, c_void_p, c_void_p] + [c_int] * 8 + \
    [c_float, c_float, c_float, c_int, c_void_p, ctypes.c_size_t, c_void_p, c_int, c_void_p, c_void_p,
     c_void_p]
LIB.mcROIPooling.argtypes = [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int,
                             c_float, c_void_p, c_void_p, c_void_p]
LIB.mcPSROIPooling.argtypes = [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float,
                               c_void_p, c_void_p, c_void_p]
LIB.mcUnary.argtypes = [c_int, c_void_p, c_void_p, c_long, c_float, c_float, c_float, c_void_p]
LIB.mcPReLU.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p]
LIB.mcLRNAcrossChannels.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                    c_float, c_float, c_void_p]
LIB.mcLRNWithinChannel.argtypes = [c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_float, c_float,
                                   c_void_p]
LIB.mcArgMax.argtypes = [c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p]
LIB.mcReduction.argtypes = [c_int, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]
LIB.mcMVN.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]
LIB.mcGatherRows.argtypes = [c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p, c_void_p]
LIB.mcCrop.argtypes = [c_void_p, c_void_p, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                       ctypes.POINTER(c_int), c_void_p]
LIB.mcTile.argtypes = [c_void_p, c_void_p, c_long, c_int, c_int, c_void_p]
LIB.mcProposalWorkspaceSize.argtypes = [c_int, c_int, c_int, ctypes.POINTER(ctypes.c_size_t)]
LIB.mcProposal.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                           c_float, c_int, c_int, c_float, c_void_p, ctypes.c_size_t, c_void_p,
                           c_void_p, c_void_p, c_void_p, c_void_p]
LIB.mcProposalHead.argtypes = LIB.mcProposal.argtypes
LIB.mcProposalRest.argtypes = LIB.mcProposal.argtypes
LIB.mcProposalTimingEnable.argtypes = [c_int]
LIB.mcProposalForceGeneralReplay.argtypes = [c_int]
LIB.mcProposalTimingCollect.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_long)]
LIB.mcProposalStatic.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                 c_float, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p]

LIB.mcConvPlanCreate.argtypes = [ctypes.POINTER(ConvGeom), ctypes.POINTER(c_void_p)]
LIB.mcConvPlanDestroy.argtypes = [c_void_p]
LIB.mcConvPlanOutputShape.argtypes = [c_void_p, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]
LIB.mcConvPlanSetWeights.argtypes = [c_void_p, c_void_p, c_void_p]
LIB.mcConvForward.argtypes = [c_void_p, c_int, c_void_p, c_void_p, ctypes.POINTER(Epilogue),
                              c_void_p]
LIB.mcConvForwardTwoTops.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p,
                                     ctypes.POINTER(Epilogue), c_void_p]
LIB.mcConvPlanFlops.argtypes = [c_void_p, c_int]
LIB.mcConvPlanFlops.restype = ctypes.c_double
LIB.mcConvPlanKernelName.argtypes = [c_void_p, c_int]
LIB.mcConvPlanKernelName.restype = ctypes.c_char_p
LIB.mcConvPlanForceConfig.argtypes = [c_void_p, c_int]
LIB.mcConvPlanForceSplit.argtypes = [c_void_p, c_int]
LIB.mcConvPlanForceWinograd.argtypes = [c_void_p, c_int]
LIB.mcConvWinogradDefault.argtypes = [c_int]
LIB.mcConvPlanForceChunk.argtypes = [c_void_p, c_int]


def conv_geom(cin, h, w, cout, kernel, stride=1, pad=0, dilation=1, group=1, transposed=False):
    def two(v):
        return (v, v) if isinstance(v, int) else tuple(v)
    kh, kw = two(kernel)
    sh, sw = two(stride)
    ph, pw = two(pad)
    dh, dw = two(dilation)
    return ConvGeom(cin, h, w, cout, kh, kw, sh, sw, ph, pw, dh, dw, group, int(transposed))


class ConvPlan(object):
    """Owns one mcConvPlan."""

    def __init__(self, geom):
        self.geom = geom
        self.handle = c_void_p()
        check_mc(LIB.mcConvPlanCreate(ctypes.byref(geom), ctypes.byref(self.handle)))

    def close(self):
        if self.handle:
            LIB.mcConvPlanDestroy(self.handle)
            self.handle = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def output_shape(self):
        ho, wo = c_int(), c_int()
        check_mc(LIB.mcConvPlanOutputShape(self.handle, ctypes.byref(ho), ctypes.byref(wo)))
        return ho.value, wo.value

    def set_weights(self, w_ptr, stream=0):
        check_mc(LIB.mcConvPlanSetWeights(self.handle, w_ptr, stream))

    def force_config(self, idx):
        check_mc(LIB.mcConvPlanForceConfig(self.handle, idx))

    def force_split(self, slices):
        check_mc(LIB.mcConvPlanForceSplit(self.handle, slices))

    def force_winograd(self, mode):
        """-1: the library decides by size, 0: direct path, 1: Winograd whenever the geometry allows."""
        check_mc(LIB.mcConvPlanForceWinograd(self.handle, mode))

    def force_chunk(self, images):
        check_mc(LIB.mcConvPlanForceChunk(self.handle, images))

    def forward(self, num, x_ptr, y_ptr, scale=None, shift=None, residual=None,
                activation=ACT_NONE, negative_slope=0.0, stream=0):
        ep = Epilogue(scale, shift, residual, activation, negative_slope)
        check_mc(LIB.mcConvForward(self.handle, num, x_ptr, y_ptr, ctypes.byref(ep), stream))

    def forward_two_tops(self, num, x_ptr, first_ptr, channels_first, second_ptr,
                         scale=None, shift=None, activation=ACT_NONE, negative_slope=0.0, stream=0):
        ep = Epilogue(scale, shift, None, activation, negative_slope)
        check_mc(LIB.mcConvForwardTwoTops(self.handle, num, x_ptr, first_ptr, channels_first,
                                          second_ptr, ctypes.byref(ep), stream))

    def flops(self, num):
        return LIB.mcConvPlanFlops(self.handle, num)

    def kernel_name(self, num):
        return LIB.mcConvPlanKernelName(self.handle, num).decode()
