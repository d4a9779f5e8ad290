"""The convolutional front end of the reference's acoustic model, as a module.

`ConvStack` builds the layer list the way ``AcousticModel.__init__`` does
(models.py:277-339): per-layer stride / dilation / padding and, above all, the
extra output length ``r = expected - valid`` that pins every layer's output
size to ``input // factor`` (models.py:292-327; without it a stack of Mellin
layers shrinks to nothing after a few layers), and applies it the way
``AcousticModel.forward`` does (models.py:423-437): non-linearity after every
layer.  Two things go beyond the reference, both optional and off by default:
more than one input channel (the reference feeds one channel of windows; a
fbank batch with deltas has three), and a frequency max-pool after chosen
layers.  Layers are this package's `MCorrLCorr` (Mellin x linear) or
`LCorrLCorr` (linear x linear, in place of the reference's
``torch.nn.Conv2d``, models.py:329-338, with the same padding rule).
"""
from typing import Callable, List, Optional, Sequence, Tuple

import torch

import mconv
import _mellin_hip as _hip

__all__ = ["ConvStackParams", "ConvStack", "FrameClassifier", "layer_plan", "pack_windows"]


class _FreqMaxPool(torch.autograd.Function):
    """max_pool2d(x, (1, 2)) for dense float32 or float16 GPU tensors through the library's pair kernels:
    one byte per output is kept for the backward pass instead of PyTorch's 8-byte indices."""

    @staticmethod
    def forward(ctx, x):
        y, which = _hip.pool_pairs_forward(x.contiguous())
        ctx.save_for_backward(which)
        ctx.f = x.shape[-1]
        return y

    @staticmethod
    def backward(ctx, grad_y):
        (which,) = ctx.saved_tensors
        return _hip.pool_pairs_backward(grad_y.contiguous(), which, ctx.f)


def freq_max_pool(x: torch.Tensor) -> torch.Tensor:
    """Maximum over pairs of neighbouring frequency bins, ``max_pool2d(x, (1, 2))``."""
    if x.is_cuda and x.dtype in (torch.float32, torch.float16):
        return _FreqMaxPool.apply(x)
    return torch.nn.functional.max_pool2d(x, (1, 2))


class ConvStackParams:
    """The convolutional fields of ``AcousticModelParams`` (models.py:45-118)."""

    def __init__(self, layers: int = 5, mellin: bool = True, kernel_time: int = 5, kernel_freq: int = 3,
                 initial_channels: int = 64, factor_schedule: int = 2, channel_factor: int = 1,
                 time_factor: int = 2, freq_factor: int = 1,
                 nonlinearity: Callable[[torch.Tensor], torch.Tensor] = torch.relu,
                 in_channels: int = 1, freq_pool_after: Sequence[int] = (), seed: Optional[int] = None):
        self.layers, self.mellin = layers, mellin
        self.kernel_time, self.kernel_freq = kernel_time, kernel_freq
        self.initial_channels, self.factor_schedule = initial_channels, factor_schedule
        self.channel_factor, self.time_factor, self.freq_factor = channel_factor, time_factor, freq_factor
        self.nonlinearity = nonlinearity
        self.in_channels = in_channels
        self.freq_pool_after = tuple(freq_pool_after)     # 1-based layer numbers followed by max_pool (1, 2)
        self.seed = seed


def layer_plan(params: ConvStackParams, time_dim: int, freq_dim: int) -> List[dict]:
    """Per-layer geometry by the rule of models.py:277-339.

    Returns one dict per layer: in/out channels, kernel, s, d, p, r and the
    output extent (after the optional frequency pool)."""
    x, y = time_dim, freq_dim
    kx, ky = params.kernel_time, params.kernel_freq
    ci, co = params.in_channels, params.initial_channels
    up_c, decim_x, on_sy = params.channel_factor, params.time_factor, params.freq_factor
    px, py = (kx - 1) // 2, (ky - 1) // 2
    off_s = dy = off_dx = 1
    if params.mellin:
        on_sx, on_dx = 1, (decim_x - 1) * kx + 1
    else:
        on_sx, on_dx = decim_x, 1
    plan = []
    for layer_no in range(1, params.layers + 1):
        if layer_no % params.factor_schedule:             # "off": output size unchanged
            dx, sx, sy, Dx, Dy = off_dx, off_s, off_s, 1, 1
        else:                                             # "on": output size divided
            dx, sx, sy, co, Dx, Dy = on_dx, on_sx, on_sy, up_c * co, decim_x, on_sy
        if params.mellin:
            new_x = mconv.mcorr_valid_size(kx, x, sx, dx, px)
            rx = max(x // Dx, 1) - new_x
            new_y = mconv.lcorr_valid_size(ky, y, sy, dy, py)
            ry = max(y // Dy, 1) - new_y
            lay = dict(kind="mcorrlcorr", p=(px, py), r=(rx, ry))
            x, y = new_x + rx, new_y + ry
        else:
            # torch.nn.Conv2d with symmetric padding (px_, py_): left padding p, right padding r
            px_ = px if (x + 2 * px - kx) // sx + 1 > 0 else px + 1
            py_ = py if (y + 2 * py - ky) // sy + 1 > 0 else py + 1
            out_x, out_y = (x + 2 * px_ - kx) // sx + 1, (y + 2 * py_ - ky) // sy + 1
            rx = out_x - mconv.lcorr_valid_size(kx, x, sx, dx, px_)
            ry = out_y - mconv.lcorr_valid_size(ky, y, sy, dy, py_)
            lay = dict(kind="lcorrlcorr", p=(px_, py_), r=(rx, ry))
            x, y = out_x, out_y
        lay.update(in_channels=ci, out_channels=co, kernel=(kx, ky), s=(sx, sy), d=(dx, dy),
                   pool=layer_no in params.freq_pool_after)
        if lay["pool"]:
            y = y // 2
        lay["out_size"] = (x, y)
        if x <= 0 or y <= 0:
            raise ValueError("layer %d of the stack has an empty output (%d x %d)" % (layer_no, x, y))
        plan.append(lay)
        ci = co
    return plan


def pack_windows(x: torch.Tensor, lens: torch.Tensor, window_size: int, window_stride: int):
    """Feature batch ``(N, T, F)`` with lengths -> the windows the convolutions see.

    As ``AcousticModel.forward`` (models.py:395-411): pad ``window_size - 1`` frames at the
    end, cut windows of ``window_size`` frames every ``window_stride``, keep only the
    ``(len - 1) // stride + 1`` windows of each utterance that start on a real frame, and fuse
    utterance and window index (time-major, as ``pack_padded_sequence`` orders them).  Returns
    the windows ``(N', 1, window_size, F)``, the convolution stack's input, and the
    ``PackedSequence`` whose ``batch_sizes`` / ``unsorted_indices`` undo the packing."""
    if window_size > 1:
        x = torch.nn.functional.pad(x, (0, 0, 0, window_size - 1))
    windows = x.unfold(1, window_size, window_stride).transpose(2, 3)      # (N, T', w, F)
    lens_ = torch.div(lens - 1, window_stride, rounding_mode="trunc") + 1
    packed = torch.nn.utils.rnn.pack_padded_sequence(windows, lens_.cpu(), batch_first=True,
                                                     enforce_sorted=False)
    return packed.data.unsqueeze(1).contiguous(), packed


class ConvStack(torch.nn.Module):
    """``x (N, C_in, T, F) -> (N, C_out, T', F')`` through the planned layers."""

    def __init__(self, time_dim: int, freq_dim: int, params: ConvStackParams):
        super().__init__()
        self.params = params
        self.plan = layer_plan(params, time_dim, freq_dim)
        self.convs = torch.nn.ModuleList()
        for lay in self.plan:
            cls = mconv.MCorrLCorr if lay["kind"] == "mcorrlcorr" else mconv.LCorrLCorr
            self.convs.append(cls(lay["in_channels"], lay["out_channels"], lay["kernel"], s=lay["s"],
                                  d=lay["d"], p=lay["p"], r=lay["r"]))
        if params.seed is not None:
            self.reset_parameters()

    @property
    def out_channels(self) -> int:
        return self.plan[-1]["out_channels"]

    @property
    def out_size(self) -> Tuple[int, int]:
        return self.plan[-1]["out_size"]

    def reset_parameters(self) -> None:
        if self.params.seed is not None:
            torch.manual_seed(self.params.seed)
        for conv in self.convs:
            conv.reset_parameters()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # ReLU, the reference's default (models.py:96-101), is applied by the convolution
        # kernel itself on the way out; any other callable runs as a pass of its own
        fused = self.params.nonlinearity in (torch.relu, torch.nn.functional.relu)
        for lay, conv in zip(self.plan, self.convs):
            x = conv(x, activation="relu") if fused else self.params.nonlinearity(conv(x))
            if lay["pool"]:
                x = freq_max_pool(x)
        return x


class FrameClassifier(torch.nn.Module):
    """Convolution stack, then a linear projection of every frame's features to log-probabilities.

    The output stage of the reference's acoustic model without its recurrent layers
    (models.py:437-454: the convolutional features of a frame, channels x bins flattened, go
    through ``torch.nn.Linear`` to ``target_dim`` scores): ``x (N, C_in, T, F) ->
    (N, T', n_out)`` log-probabilities.  The projection is PyTorch's; only the convolutions
    run in this package's kernels."""

    def __init__(self, stack: ConvStack, n_out: int = 62):
        super().__init__()
        self.stack = stack
        self.out = torch.nn.Linear(stack.out_channels * stack.out_size[1], n_out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        h = self.stack(x)                                   # (N, C, T', F')
        h = h.permute(0, 2, 1, 3).flatten(2)                # (N, T', C * F')
        return torch.nn.functional.log_softmax(self.out(h), dim=-1)
