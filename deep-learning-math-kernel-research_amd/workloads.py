"""The configured int8 layers (ResNet-50 / VGG-16 / MobileNet-v2 shapes) with their operation and
byte accounting, and synthetic-tensor setup on the device.

Operations follow the reference's benchmark accounting (tests/elt_conv_utils.cpp:638-659):
2 x multiply-accumulates of the DIRECT algorithm with padded taps left out -- so Winograd figures
are "effective" TOPS.  Algorithmic bytes = every user tensor touched once (input, packed s8
weights, output, sum operand, per-channel f32 scale + shift); Winograd intermediates are not
algorithmic.
"""
import math

from . import (CONV_DIRECT, CONV_DIRECT_1X1, CONV_WINOGRAD, EL_NO_CALI, F32, FLT_MAX, NCHW16C, NHWC, S8, U8, Conv,
               make_desc, up16, wino_tinput_range)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s


class Workload:
    def __init__(self, key, title, n, ic, oc, hw, k=1, pad=0, stride=1, algorithm=CONV_DIRECT, in_type=U8,
                 out_type=U8, with_sum=False, depthwise=False, w_sigma=0.05, T=0, relu6=False, nhwc=False, oh=None, in_z=0.0, nhwc_out=False,
                 nhwc_in=False, tile=6):
        self.key, self.title = key, title
        self.n, self.ic, self.oc, self.hw, self.k, self.pad, self.stride = n, ic, oc, hw, k, pad, stride
        self.algorithm, self.in_type, self.out_type = algorithm, in_type, out_type
        self.with_sum, self.depthwise, self.w_sigma, self.T, self.relu6 = with_sum, depthwise, w_sigma, T, relu6
        self.tile = tile   # Winograd tile size: 6 = F(4x4,3x3), 4 = F(2x2,3x3), 5 = F(3x3,3x3)
        self.in_z = in_z   # input zero point (the reference's "...z" data-type configurations)
        self.nhwc = nhwc   # activations [n][h][w][c] on both sides instead of nChw16c
        self.nhwc_in, self.nhwc_out = nhwc or nhwc_in, nhwc or nhwc_out
        # oh given: the right / bottom pads are whatever that output size needs (src/elx_conv.cpp:36-37)
        self.oh = oh if oh is not None else (hw + 2 * pad - k) // stride + 1

    # 2 * MACs, padded taps excluded
    def ops(self):
        def valid(o_len, i_len):
            tot = 0
            for o in range(o_len):
                for kk in range(self.k):
                    i = o * self.stride + kk - self.pad
                    tot += 0 <= i < i_len
            return tot
        v = valid(self.oh, self.hw)
        per_pair = v * v
        g = self.ic if self.depthwise else 1
        return 2.0 * self.n * per_pair * (self.ic // g) * self.oc

    def algorithmic_bytes(self):
        esz = {U8: 1, S8: 1, F32: 4}
        # nhwc input with at most four channels is compact (a first layer's image)
        n_in = self.n * (self.ic if self.nhwc_in and self.ic <= 4 else up16(self.ic)) * self.hw * self.hw
        if self.stride == 2 and self.k == 1:
            n_in //= 4  # a stride-2 1x1 only samples every other row and column
        n_out = self.n * up16(self.oc) * self.oh * self.oh
        if self.depthwise:
            w = up16(self.oc) * 9
        elif self.algorithm == CONV_WINOGRAD:
            w = self.tile * self.tile * up16(self.ic) * up16(self.oc)
        else:
            w = up16(self.ic) * up16(self.oc) * self.k * self.k
        b = n_in * esz[self.in_type] + w + n_out * esz[self.out_type] + 8 * up16(self.oc)
        if self.with_sum:
            b += n_out * esz[self.out_type]
        return float(b)

    def bound(self):
        t_mfma = self.ops() / (PEAK_INT8_TOPS * 1e12)
        t_hbm = self.algorithmic_bytes() / (PEAK_HBM_GBS * 1e9)
        return ("mfma", t_mfma) if t_mfma >= t_hbm else ("hbm", t_hbm)

    def descriptor(self, out_quant=None, sum_scale=None, tinput_quant=(EL_NO_CALI, EL_NO_CALI)):
        """out_quant = (scale, z) and sum_scale as calibrated (DeviceLayer); left out, an analytic estimate
        stands in: four sigmas of the pre-activation over the code range, and 0.7 for the sum operand."""
        fan = self.k * self.k * (1 if self.depthwise else self.ic)
        if out_quant is None:
            # u8 in [0,255]/255 ~ U[0,1): E[x^2] = 1/3
            out_quant = (4.0 * self.w_sigma * math.sqrt(fan / 3.0) / (127.0 if self.out_type == S8 else 255.0), 0.0)
        out_scale, out_z = out_quant
        if sum_scale is None:
            sum_scale = 0.7
        relu = (0.0, FLT_MAX)
        if self.relu6:
            out_scale = 6.0 / 255.0
            relu = (0.0, 255.0)   # ReLU6 in the quantized output domain
        if self.out_type == S8:
            relu = (0.0, 127.0)
        g = self.ic if self.depthwise else 1
        d = make_desc(self.n, self.ic, self.oc, self.hw, self.hw, self.k, self.k, self.pad, self.stride, g=g,
                      algorithm=self.algorithm, input_type=self.in_type, output_type=self.out_type,
                      with_bias=True, with_relu=True, with_ip_sum=self.with_sum,
                      input_quant=(1.0, 0.0) if self.in_type == F32 else (1.0 / 255.0, self.in_z),
                      output_quant=(out_scale, out_z), sum_quant=(sum_scale, 0.0) if self.with_sum else (0.0, 0.0),
                      wino_tinput_quant=tinput_quant, relu_bound=relu, flatting_t=self.T,
                      tile_size=self.tile if self.algorithm == CONV_WINOGRAD else 0,
                      execution_mode=0xa161 if self.algorithm == CONV_WINOGRAD else 0)
        if self.nhwc_in:
            d.input_fmt = NHWC
        if self.nhwc_out:
            d.output_fmt = NHWC
        if d.oh != self.oh:
            d.oh = d.ow = self.oh
            d.pad_r = d.pad_b = max(0, (self.oh - 1) * self.stride + self.k - self.hw - self.pad)
        return d


WORKLOADS = {w.key: w for w in [
    Workload("C1", "1x1 64->256 @56x56 N=1, ReLU, f32 out (ResNet-50 res2 expand)", 1, 64, 256, 56, out_type=F32),
    Workload("C2", "3x3 128->128 @28x28 N=32 pad 1, bias+ReLU, u8 out (ResNet-50 res3)", 32, 128, 128, 28, k=3, pad=1,
             T=14),
    Workload("C3a", "1x1 1024->256 @14x14 N=64, sum+ReLU, s8 out (ResNet-50 res4 reduce)", 64, 1024, 256, 14,
             algorithm=CONV_DIRECT_1X1, out_type=S8, with_sum=True),
    Workload("C3b", "1x1 s2 512->1024 28x28->14x14 N=64, sum+ReLU, s8 out (ResNet-50 res4 projection)", 64, 512, 1024,
             28, stride=2, algorithm=CONV_DIRECT_1X1, out_type=S8, with_sum=True),
    # the same two layers with nhwc activations, as the reference's tuned ResNet-v1.5 run feeds them
    # (scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh:62 "--input-format=nhwc --output-format=nhwc")
    Workload("C3a_nhwc", "1x1 1024->256 @14x14 N=64, sum+ReLU, s8 out, nhwc activations", 64, 1024, 256, 14,
             algorithm=CONV_DIRECT_1X1, out_type=S8, with_sum=True, nhwc=True),
    Workload("C3b_nhwc", "1x1 s2 512->1024 28x28->14x14 N=64, sum+ReLU, s8 out, nhwc activations", 64, 512, 1024,
             28, stride=2, algorithm=CONV_DIRECT_1X1, out_type=S8, with_sum=True, nhwc=True),
    # stride-2 layers of the reference's tuned int8 runs
    # (scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh conv2d_13: pre-padded 58x58 input;
    #  scripts/best_configs/mobilenetv1-n64-clx-1s-int8.sh Conv2d_4_depthwise: pad only right / bottom)
    Workload("R13", "3x3 s2 128->128 58x58->28x28 N=64 pad 0, bias+ReLU, s8 out (ResNet-50 v1.5 conv2d_13)", 64, 128, 128,
             58, k=3, pad=0, stride=2, out_type=S8, T=14),
    # ResNet-50's first layer with the zero-point input configuration of the tuned run
    # (scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh:12 "U8F32S8F32z"), here on nChw16c input:
    # the three channels occupy one 16-channel unit per tap
    Workload("R1", "7x7 s2 3->64 224x224->112x112 N=64 pad 3, 3-channel nhwc input with zero point 128, bias+ReLU, "
             "s8 nhwc out (ResNet-50 conv1)", 64, 3, 64, 224, k=7, pad=3, stride=2, out_type=S8, T=14, in_z=128.0,
             nhwc_in=True, nhwc_out=True),
    Workload("M1", "3x3 s2 3->32 224x224->112x112 N=64 pads right/bottom, 3-channel nhwc input with zero point 128, "
             "bias+ReLU, s8 out (MobileNet-v1 Conv__224)", 64, 3, 32, 224, k=3, pad=0, stride=2, out_type=S8, T=14,
             in_z=128.0, oh=112, nhwc_in=True),
    Workload("M4", "depthwise 3x3 s2 C=128 56x56->28x28 N=64, bias+ReLU6, u8 out (MobileNet-v1 Conv2d_4)", 64, 128, 128,
             56, k=3, pad=0, stride=2, depthwise=True, w_sigma=0.1, T=28, relu6=True, oh=28),
    Workload("C4a", "Winograd F(4,3) 256->256 @56x56 N=64, fp32 in/out (VGG-16 conv3)", 64, 256, 256, 56, k=3, pad=1,
             algorithm=CONV_WINOGRAD, in_type=F32, out_type=F32, w_sigma=0.02),
    Workload("C4b", "Winograd F(4,3) 512->512 @28x28 N=64, fp32 in/out (VGG-16 conv4)", 64, 512, 512, 28, k=3, pad=1,
             algorithm=CONV_WINOGRAD, in_type=F32, out_type=F32, w_sigma=0.02),
    # the same two layers as the reference's tuned VGG int8 run feeds them: u8 in, s8 out
    # (scripts/best_configs/vgg-n64-8180-1s-int8.sh:9,28,36 "--data-type-cfg=U8F32S8F32")
    Workload("C4a_i8", "Winograd F(4,3) 256->256 @56x56 N=64, u8 in / s8 out (VGG-16 conv3, U8F32S8F32)", 64, 256, 256, 56,
             k=3, pad=1, algorithm=CONV_WINOGRAD, in_type=U8, out_type=S8, w_sigma=0.02),
    Workload("C4b_i8", "Winograd F(4,3) 512->512 @28x28 N=64, u8 in / s8 out (VGG-16 conv4, U8F32S8F32)", 64, 512, 512, 28,
             k=3, pad=1, algorithm=CONV_WINOGRAD, in_type=U8, out_type=S8, w_sigma=0.02),
    Workload("C4b_i8_t4", "Winograd F(2,3) (tile size 4) 512->512 @28x28 N=64, u8 in / s8 out", 64, 512, 512, 28,
             k=3, pad=1, algorithm=CONV_WINOGRAD, in_type=U8, out_type=S8, w_sigma=0.02, tile=4),
    Workload("C4b_i8_t5", "Winograd F(3,3) (tile size 5) 512->512 @28x28 N=64, u8 in / s8 out", 64, 512, 512, 28,
             k=3, pad=1, algorithm=CONV_WINOGRAD, in_type=U8, out_type=S8, w_sigma=0.02, tile=5),
    Workload("C5a", "depthwise 3x3 C=144 @56x56 N=64, bias+ReLU6, u8 out (MobileNet-v2)", 64, 144, 144, 56, k=3, pad=1,
             depthwise=True, w_sigma=0.1, T=14, relu6=True),
    Workload("C5b", "depthwise 3x3 C=960 @7x7 N=64, bias+ReLU6, u8 out (MobileNet-v2)", 64, 960, 960, 7, k=3, pad=1,
             depthwise=True, w_sigma=0.1, T=7, relu6=True),
]}


def _L(count, key, title, n, ic, oc, hw, **kw):
    """one distinct layer shape of a network and how many of the network's layers have it"""
    return count, Workload(key, title, n, ic, oc, hw, **kw)


def _pw(count, name, ic, oc, hw, stride=1, nhwc_in=False, nhwc_out=False, n=64, out_type=S8, algorithm=CONV_DIRECT_1X1):
    w = Workload(name, "1x1%s %d->%d @%d" % (" s2" if stride == 2 else "", ic, oc, hw), n, ic, oc, hw, stride=stride,
                 algorithm=algorithm, out_type=out_type)
    w.nhwc_in, w.nhwc_out = nhwc_in, nhwc_out
    return count, w


def _wino(count, name, ic, oc, hw):
    return _L(count, name, "Winograd F(4,3) %d->%d @%d u8->s8" % (ic, oc, hw), 64, ic, oc, hw, k=3, pad=1,
              algorithm=CONV_WINOGRAD, in_type=U8, out_type=S8, w_sigma=0.02)


def _dw(count, name, c, hw, stride):
    if stride == 1:
        return _L(count, name, "depthwise 3x3 C=%d @%d" % (c, hw), 64, c, c, hw, k=3, pad=1, depthwise=True, w_sigma=0.1,
                  T=min(hw, 28), relu6=True, out_type=U8)
    return _L(count, name, "depthwise 3x3 s2 C=%d %d->%d" % (c, hw, hw // 2), 64, c, c, hw, k=3, pad=0, stride=2,
              depthwise=True, w_sigma=0.1, T=min(hw // 2, 28), relu6=True, oh=hw // 2, out_type=U8)


# The convolution layers of the reference's tuned int8 model runs, batch 64, as (count, layer shape):
# shapes, strides, pads, data types and activation layouts follow the command lines of
#   scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh   (ResNet-50 v1.5: 53 convolutions + the FC layer)
#   scripts/best_configs/mobilenetv1-n64-clx-1s-int8.sh  (MobileNet-v1: 27 convolutions + the FC layer)
#   scripts/best_configs/vgg-n64-8180-1s-int8.sh         (VGG-19 without conv1_1: 15 convolutions)
# and the counts follow the layer names listed above each command there.  One deviation: MobileNet's FC
# (1001 output channels) writes nChw16c where the script asks for nhwc.
NETWORKS = {
    "resnet50_v1_5_int8": [
        _L(1, "conv2d", "7x7 s2 3->64 224->112 pad 3, 3-channel nhwc in, zero point 128, nhwc out", 64, 3, 64, 224, k=7,
           pad=3, stride=2, out_type=S8, T=14, in_z=128.0, nhwc_in=True, nhwc_out=True),
        _wino(3, "conv2d_3", 64, 64, 56), _wino(3, "conv2d_16", 128, 128, 28), _wino(5, "conv2d_29", 256, 256, 14),
        _wino(2, "conv2d_48", 512, 512, 7),
        _L(1, "conv2d_13", "3x3 s2 128->128 58->28", 64, 128, 128, 58, k=3, stride=2, out_type=S8, T=14),
        _L(1, "conv2d_26", "3x3 s2 256->256 30->14", 64, 256, 256, 30, k=3, stride=2, out_type=S8, T=14),
        _L(1, "conv2d_45", "3x3 s2 512->512 16->7", 64, 512, 512, 16, k=3, stride=2, out_type=S8, T=7),
        _pw(1, "conv2d_11", 256, 512, 56, stride=2), _pw(1, "conv2d_24", 512, 1024, 28, stride=2),
        _pw(1, "conv2d_43", 1024, 2048, 14, stride=2),
        _pw(1, "conv2d_2", 64, 64, 56), _pw(4, "conv2d_1", 64, 256, 56), _pw(2, "conv2d_5", 256, 64, 56),
        _pw(1, "conv2d_12", 256, 128, 56),
        _pw(4, "conv2d_14", 128, 512, 28), _pw(3, "conv2d_15", 512, 128, 28, nhwc_out=True), _pw(1, "conv2d_25", 512, 256, 28),
        _pw(6, "conv2d_27", 256, 1024, 14, nhwc_out=True), _pw(5, "conv2d_28", 1024, 256, 14, nhwc_in=True, nhwc_out=True),
        _pw(1, "conv2d_44", 1024, 512, 14, nhwc_in=True, nhwc_out=True),
        _pw(3, "conv2d_46", 512, 2048, 7, nhwc_out=True), _pw(2, "conv2d_47", 2048, 512, 7, nhwc_in=True, nhwc_out=True),
        _pw(1, "FC", 2048, 1008, 8, nhwc_in=True, nhwc_out=True, n=1, out_type=F32, algorithm=CONV_DIRECT),
    ],
    "mobilenet_v1_int8": [
        _L(1, "Conv__224", "3x3 s2 3->32 224->112, pads right/bottom, 3-channel nhwc in, zero point 128", 64, 3, 32, 224,
           k=3, pad=0, stride=2, out_type=S8, T=14, in_z=128.0, oh=112, nhwc_in=True),
        _pw(1, "Conv__226", 32, 64, 112), _pw(1, "Conv__228", 64, 128, 56), _pw(1, "Conv__230", 128, 128, 56),
        _pw(1, "Conv__232", 128, 256, 28), _pw(1, "Conv__234", 256, 256, 28), _pw(1, "Conv__236", 256, 512, 14),
        _pw(5, "Conv__238", 512, 512, 14), _pw(1, "Conv__248", 512, 1024, 7), _pw(1, "Conv__250", 1024, 1024, 7, nhwc_out=True),
        _pw(1, "Conv__252", 1024, 1001, 8, nhwc_in=True, n=1, out_type=F32, algorithm=CONV_DIRECT),
        _dw(1, "Conv2d_1_depthwise", 32, 112, 1), _dw(1, "Conv2d_2_depthwise", 64, 112, 2), _dw(1, "Conv2d_3_depthwise", 128, 56, 1),
        _dw(1, "Conv2d_4_depthwise", 128, 56, 2), _dw(1, "Conv2d_5_depthwise", 256, 28, 1), _dw(1, "Conv2d_6_depthwise", 256, 28, 2),
        _dw(5, "Conv2d_7_depthwise", 512, 14, 1), _dw(1, "Conv2d_12_depthwise", 512, 14, 2), _dw(1, "Conv2d_13_depthwise", 1024, 7, 1),
    ],
    "vgg19_int8": [
        _wino(1, "conv1_2", 64, 64, 224), _wino(1, "conv2_1", 64, 128, 112), _wino(1, "conv2_2", 128, 128, 112),
        _wino(1, "conv3_1", 128, 256, 56), _wino(3, "conv3_2", 256, 256, 56), _wino(1, "conv4_1", 256, 512, 28),
        _wino(3, "conv4_2", 512, 512, 28), _wino(4, "conv5_1", 512, 512, 14),
    ],
}


# ---- synthetic tensors: a self-contained generator, so that a seed gives the same bytes on every host -------
_GAMMA = 0x9E3779B97F4A7C15


def splitmix64(seed, count, offset=0):
    """outputs offset .. offset+count-1 of the splitmix64 sequence started at `seed` (uint64 array).  The
    state of step k is seed + (k + 1) * GAMMA, so the sequence is evaluated as a vector."""
    import numpy as np
    with np.errstate(over="ignore"):
        z = np.arange(offset + 1, offset + count + 1, dtype=np.uint64)
        z *= np.uint64(_GAMMA)
        z += np.uint64(seed)
        z ^= z >> np.uint64(30)
        z *= np.uint64(0xBF58476D1CE4E5B9)
        z ^= z >> np.uint64(27)
        z *= np.uint64(0x94D049BB133111EB)
        z ^= z >> np.uint64(31)
        return z


_last_uniform = {}


def uniform01(seed, count, offset=0):
    """U[0,1) as float32: the top 24 bits of each splitmix64 output over 2^24 (exact in float32); evaluated
    in blocks that stay in the host's cache.  The last array is kept: variants of one layer share its tensors."""
    import numpy as np
    if (seed, count, offset) in _last_uniform:
        return _last_uniform[(seed, count, offset)]
    out = np.empty(count, np.float32)
    step = 1 << 18
    for lo in range(0, count, step):
        m = min(step, count - lo)
        out[lo:lo + m] = splitmix64(seed, m, offset + lo) >> np.uint64(40)
    out *= np.float32(2.0 ** -24)
    _last_uniform.clear()
    _last_uniform[(seed, count, offset)] = out
    return out


def normal(seed, count, sigma):
    """N(0, sigma) as float32 by Box-Muller on pairs of the uniform stream (both branches used)"""
    import numpy as np
    half = (count + 1) // 2
    out = np.empty(2 * half, np.float32)
    step = 1 << 17
    for lo in range(0, half, step):
        m = min(step, half - lo)
        u = (splitmix64(seed, 2 * m, 2 * lo) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
        r = np.sqrt(-2.0 * np.log1p(-u[0::2])) * sigma          # 1 - u is in (0, 1]
        t = 2.0 * np.pi * u[1::2]
        out[2 * lo:2 * (lo + m):2] = r * np.cos(t)
        out[2 * lo + 1:2 * (lo + m):2] = r * np.sin(t)
    return out[:count]


# frozen seeds of the configured layers; every tensor of a layer takes its own stream (seed + 2^32 * index)
SEEDS = {"C1": 1001, "C2": 1002, "C3a": 1003, "C3b": 1004, "C4a": 1005, "C4b": 1006, "C5a": 1007, "C5b": 1008}


def seed_of(key):
    base = key.split("@")[0].split("_")[0]   # C3a_nhwc, C4b_i8_t4, C2@N=512 share their layer's tensors
    if base in SEEDS:
        return SEEDS[base]
    return 2000 + sum((i + 1) * ord(ch) for i, ch in enumerate(key)) % 100000


class DeviceLayer:
    """Synthetic device-resident tensors of one workload (torch owns the memory) and its prepared
    convolution handle, set up the way the reference's harness sets up a layer (tests/elt_conv_utils.cpp:
    87-463): fp32 tensors are drawn (here: seeded, U[0,1) activations, N(0, sigma) weights, N(0, 0.01)
    bias, N(0, 1) sum operand), the quantization scales are calibrated from them -- output_quant and
    sum_quant from the fp32 reference convolution (ehip_ref_conv_f32_range + ehip_calibrate_output_quant),
    wino_tinput_quant from the transformed-input range (ehip_wino_tinput_range) -- and the input and the sum
    operand are quantized with the harness's helper (ehip_quantize_input_u8).  Differences from the harness:
    the input scale is the fixed 1/255 of a U[0,1) image, u8 tensors are calibrated onto 255 codes rather
    than the harness's 127, and a ReLU6 layer keeps its 6/255 output scale."""

    def __init__(self, wl, seed=None, calibrate=True):
        import numpy as np
        import torch
        from . import (quantize_input_u8, ref_conv_f32_range, calibrate_output_quant, reorder_nchw_to_blocked,
                       reorder_oihw_to_blocked)
        self.wl = wl
        seed = seed_of(wl.key) if seed is None else seed
        ic2, oc2 = up16(wl.ic) // 16, up16(wl.oc) // 16
        few = wl.nhwc_in and wl.ic <= 4    # a first layer's compact image [n][h][w][ic]

        def stream(index):
            return seed + (index << 32)

        def blocked(t_nchw, c):            # nchw -> nChw16c on the device
            n, _, h, w = t_nchw.shape
            out = torch.empty((n, up16(c) // 16, h, w, 16), dtype=t_nchw.dtype, device="cuda")
            reorder_nchw_to_blocked(out, t_nchw, t_nchw.element_size(), n, c, h, w)
            return out

        def nhwc(t_blocked, c):            # nChw16c -> [n][h][w][c]
            n, c2, h, w, _ = t_blocked.shape
            return t_blocked.permute(0, 2, 3, 1, 4).reshape(n, h, w, c2 * 16)[..., :c].contiguous()

        # fp32 tensors; a zero point moves the image to U[0,1) - z / 255, so that its codes still cover 0..255
        in_scale = 1.0 if wl.in_type == F32 else 1.0 / 255.0
        x = torch.from_numpy(uniform01(stream(0), wl.n * wl.ic * wl.hw * wl.hw)).cuda().reshape(wl.n, wl.ic, wl.hw, wl.hw)
        if wl.in_z:
            x -= wl.in_z / 255.0
        x_f32 = blocked(x, wl.ic)
        kshape = (wl.ic, 1, wl.k, wl.k) if wl.depthwise else (wl.oc, wl.ic, wl.k, wl.k)
        w = torch.from_numpy(normal(stream(1), int(np.prod(kshape)), wl.w_sigma)).cuda().reshape(kshape)
        if wl.depthwise:
            self.w = w.reshape(wl.ic, wl.k, wl.k).contiguous()
        else:
            self.w = torch.empty((oc2, ic2, wl.k, wl.k, 16, 16), dtype=torch.float32, device="cuda")
            reorder_oihw_to_blocked(self.w, w, wl.oc, wl.ic, wl.k, wl.k)
        bias = np.zeros(oc2 * 16, np.float32)
        bias[:wl.oc] = normal(stream(2), wl.oc, 0.01)
        self.bias = torch.from_numpy(bias).cuda()
        r_f32 = None
        if wl.with_sum:
            r = torch.from_numpy(normal(stream(3), wl.n * wl.oc * wl.oh * wl.oh, 1.0)).cuda()
            r_f32 = blocked(r.reshape(wl.n, wl.oc, wl.oh, wl.oh), wl.oc)
        torch.cuda.synchronize()

        # calibration
        out_quant, sum_scale = None, 0.0
        self.calibration = {}
        if calibrate and wl.out_type != F32 and not wl.relu6:
            d32 = wl.descriptor(out_quant=(1.0, 0.0))
            d32.input_type, d32.input_fmt, d32.output_fmt = F32, NCHW16C, NCHW16C
            scratch = r_f32.clone() if wl.with_sum else None
            mn, mx = ref_conv_f32_range(d32, x_f32, self.w, self.bias, scratch)
            sum_absmax = float(r_f32.abs().max()) if wl.with_sum else 0.0
            rep = 127.0 if wl.out_type == S8 else 255.0
            s_o, z_o, sum_scale = calibrate_output_quant(d32, mn, mx, sum_absmax, rep)
            out_quant = (s_o, z_o)
            self.calibration = {"ref_out_min": mn, "ref_out_max": mx, "output_scale": s_o, "output_z": z_o,
                                "sum_scale": sum_scale if wl.with_sum else None}
            del scratch

        # user tensors
        if wl.in_type == U8:
            xq = torch.empty(x_f32.shape, dtype=torch.uint8, device="cuda")
            quantize_input_u8(xq, x_f32, x_f32.numel(), in_scale, wl.in_z)
            self.x = nhwc(xq, wl.ic) if wl.nhwc_in else xq
        else:
            self.x = nhwc(x_f32, wl.ic) if wl.nhwc_in else x_f32
        tdt = {U8: torch.uint8, S8: torch.int8, F32: torch.float32}[wl.out_type]
        oshape = (wl.n, wl.oh, wl.oh, wl.oc) if wl.nhwc_out else (wl.n, oc2, wl.oh, wl.oh, 16)
        if wl.with_sum:
            # the sum operand in the output's own type: its codes at scale max|r| / 127 (s8) or 255 (u8)
            rq = torch.empty(r_f32.shape, dtype=torch.uint8, device="cuda")
            rep = 127.0 if wl.out_type == S8 else 255.0
            quantize_input_u8(rq, r_f32, r_f32.numel(), float(r_f32.abs().max()) / rep, 0.0)
            rq = rq.view(tdt) if wl.out_type != F32 else r_f32
            self.out = nhwc(rq, wl.oc) if wl.nhwc_out else rq
        else:
            self.out = torch.zeros(oshape, dtype=tdt, device="cuda")
        del x, x_f32, w, r_f32
        tq = (EL_NO_CALI, EL_NO_CALI)
        if wl.algorithm == CONV_WINOGRAD:
            mn, mx = wino_tinput_range(wl.descriptor(tinput_quant=(1.0, 0.0)), self.x)
            mn, mx = mn * in_scale, mx * in_scale   # u8 input: the range comes back in code units
            diff = mx - mn + 1e-6
            tq = (diff / 255.0, -mn * 255.0 / diff)
            self.calibration.update({"tinput_min": mn, "tinput_max": mx})
        self.desc = wl.descriptor(out_quant=out_quant, sum_scale=sum_scale, tinput_quant=tq)
        self.conv = Conv(self.desc)
        self.conv.prepare(self.w, self.bias)
        torch.cuda.synchronize()

    def run(self, count=1):
        self.conv.execute_repeat(self.out, self.x, count, bias=self.bias)
