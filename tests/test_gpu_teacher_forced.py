"""Teacher-forced layer parity over 32 frames of delta accumulation.

The CPU oracle model runs free; every layer call it makes is recorded (inputs and outputs).
The corresponding HIP layer -- which keeps its own caches across the whole sequence -- is then
fed the oracle's inputs for that call.  With identical inputs every frame, the bar is:

  * update masks (and therefore active-pixel index sets) equal bit for bit at every layer
  * elementwise layers (sparsify, activation/truncation, add, densify) equal bit for bit
  * contractions (conv, transposed conv) within 1e-4 relative (fp32) / 2e-2 absolute (fp16; for
    values beyond +-10, where one fp16 step alone exceeds that, two steps of the value: 2^-9
    relative -- the random-init HRNet reaches +-300); global average pooling within float-sum
    reordering

Free-running models cannot be held to mask equality in fp16: one last-bit difference of a
convolution output next to a threshold legitimately flips a truncation decision.
"""
import pytest
import torch

from oracle import delta_layers as OL
from util import DEV, assert_masked_close, assert_masked_equal, cl, poison

pytestmark = pytest.mark.gpu

HOOKED = (OL.DCSparsify, OL.DCConv2d, OL.DCConvTranspose2d, OL.DCActivation, OL.DCDensify, OL.DCAdd,
          OL.DCMaxPooling, OL.DCAdaptiveAveragePooling, OL.DCUpsamplingNearest2d, OL.DCConcatenate,
          OL.DCBatchNorm2d)


def _to_gpu(v):
    """Oracle value -> HIP layer input; delta tensors get NaN at their inactive pixels."""
    if isinstance(v, tuple):
        delta, mask = v
        return cl(poison(delta, mask)), cl(mask.clone())
    return cl(v)


def _compare(kind, got, want, dtype, where):
    if isinstance(want, tuple):
        (g, gm), (w, wm) = got, want
        assert torch.equal(gm.cpu(), wm), f"{where}: {int((gm.cpu() != wm).sum())} mask words differ"
        if kind == "exact":
            assert_masked_equal(g, w, wm, where)
        elif dtype == torch.float32:
            assert_masked_close(g, w, wm, 1e-4, 1e-5, where)
        elif dtype == torch.bfloat16:  # one bfloat16 step is 2^-8 of the value
            assert_masked_close(g, w, wm, 2.0 ** -7, 2e-2, where)
        else:
            assert_masked_close(g, w, wm, 2.0 ** -9, 2e-2, where)
    else:
        if kind == "exact":
            assert torch.equal(got.cpu(), want), f"{where}: max diff {float((got.cpu().float() - want.float()).abs().max())}"
        else:
            tol = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 4e-2}[dtype]
            assert float((got.cpu().float() - want.float()).abs().max()) <= tol * max(1.0, float(want.abs().max())), where


def run_teacher_forced(ref, dut, video, dtype):
    records = []
    hooks = []
    for name, mod in ref.named_modules():
        if isinstance(mod, HOOKED):
            hooks.append(mod.register_forward_hook(
                lambda m, inp, out, name=name: records.append((name, m, inp, out))))
    dut_mods = dict(dut.named_modules())
    checked = 0
    with torch.no_grad():
        for t in range(video.shape[0]):
            records.clear()
            ref(video[t:t + 1].to(dtype))
            conv_out = {}
            for name, m, inp, out in records:
                where = f"frame {t} {name} ({type(m).__name__})"
                hip = dut_mods[name]
                if isinstance(m, (OL.DCActivation, OL.DCDensify)) and name.endswith(("activation_layer", "densify_layer")):
                    conv_out[name.rsplit(".", 1)[0]] = inp[0]  # what the owning convolution produced
                if isinstance(m, (OL.DCConv2d, OL.DCConvTranspose2d)):
                    hip.frame_idx = t
                    got = hip.conv_delta(_to_gpu(inp[0]))
                    _compare("close", got, conv_out.get(name, out), dtype, where)
                elif isinstance(m, OL.DCAdaptiveAveragePooling):
                    _compare("close", hip(_to_gpu(inp[0])), out, dtype, where)
                elif isinstance(m, (OL.DCAdd, OL.DCConcatenate)):
                    _compare("exact", hip(_to_gpu(inp[0]), _to_gpu(inp[1])), out, dtype, where)
                else:
                    _compare("exact", hip(_to_gpu(inp[0])), out, dtype, where)
                checked += 1
    for h in hooks:
        h.remove()
    return checked


def _build(builder, dtype, thr, state=None, **kw):
    from test_gpu_network import _models
    _, ref, dut = _models(builder, dtype, thr, state, **kw)
    return ref, dut


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_mobilenet_teacher_forced_32_frames(lib, dtype):
    from deltacnn_amd.video import moving_rectangles_video
    from test_gpu_network import _calibrated_state, _mobilenet
    video = moving_rectangles_video(frames=33, height=96, width=96, n_rect=2, min_size=10, max_size=30)
    ref, dut = _build(_mobilenet, dtype, 0.05, _calibrated_state(video[:4]))
    n = run_teacher_forced(ref, dut, video, dtype)
    assert n == 33 * (1 + 52 + 35 + 10 + 1 + 1)  # sparsify, convs, activations, adds, pool, densify


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_toy_cnn_teacher_forced(lib, dtype):
    from deltacnn_amd.networks import ToyCNN
    from deltacnn_amd.video import noise_block_video
    video = noise_block_video(frames=10, size=64, fraction=0.05)
    ref, dut = _build(ToyCNN, dtype, 0.05)
    assert run_teacher_forced(ref, dut, video, dtype) == 10 * (1 + 3 + 2 + 1)


@pytest.mark.parametrize("network", ["hrnet", "dla34"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_multibranch_teacher_forced(lib, network, dtype):
    """Every layer call of HRNet (strided exchange convolutions, nearest upsampling, chained sums
    with ReLU) and of DLA-34 + CenterNet heads (max-pooling, concatenating roots, transposed
    convolutions, dense heads) over 8 frames, each HIP layer fed the oracle's inputs."""
    from deltacnn_amd.video import moving_rectangles_video
    from test_gpu_network import _calibrated, _dla, _hrnet
    builder, size = {"hrnet": (_hrnet, (64, 64)), "dla34": (_dla, (64, 96))}[network]
    video = moving_rectangles_video(frames=8, height=size[0], width=size[1], n_rect=2, min_size=8, max_size=24)
    ref, dut = _build(builder, dtype, 0.05, _calibrated(builder, video[:3]))
    n = run_teacher_forced(ref, dut, video, dtype)
    assert n % 8 == 0 and n // 8 > 100


# --------------------------------------------------------------------------------------------
# The measured configurations at their real sizes, fp16 (the type they are measured in)
# --------------------------------------------------------------------------------------------
def test_mobilenet_224_fp16_teacher_forced_34_frames(lib):
    """MobileNetV2 w1.0 at 224x224, fp16, on the synthetic clip of the headline configuration
    (smooth-noise background, three textured rectangles moving 1-4 px per frame, sensor noise
    sigma 0.01, threshold 0.05 on all layers): 34 frames, every layer call of every frame fed the
    CPU oracle's input.  Masks bit for bit, elementwise layers bit for bit, convolutions within
    2e-2 absolute -- after 33 frames of delta accumulation in every layer's caches."""
    from deltacnn_amd.networks import MobileNetV2
    from deltacnn_amd.video import moving_rectangles_video
    from test_gpu_network import _calibrated
    video = moving_rectangles_video(frames=34)  # the generator's defaults are that configuration
    assert tuple(video.shape[1:]) == (3, 224, 224)

    def full(L, **kw):
        return MobileNetV2(L, **kw)  # 1000-way head
    ref, dut = _build(full, torch.float16, 0.05, _calibrated(full, video[:3]))
    n = run_teacher_forced(ref, dut, video, torch.float16)
    assert n == 34 * (1 + 52 + 35 + 10 + 1 + 1)


@pytest.mark.parametrize("network", ["hrnet_w32", "dla34_centernet"])
def test_full_depth_networks_fp16_teacher_forced(lib, network):
    """HRNet-W32 (full depth: 1 / 4 / 3 modules of 4 blocks, 17 heat maps) at 256x256 and DLA-34 +
    CenterNet heads (80 classes, 256-channel heads) at 544x960, fp16, threshold 0.05: every layer
    call of 5 resp. 4 frames fed the CPU oracle's input, bar as above."""
    from deltacnn_amd.networks import DLA34CenterNet, HRNet
    from deltacnn_amd.video import moving_rectangles_video
    from test_gpu_network import _calibrated
    if network == "hrnet_w32":
        builder, frames = HRNet, 5
        video = moving_rectangles_video(frames=frames, height=256, width=256, n_rect=1, min_size=100,
                                        max_size=180, min_speed=2, max_speed=6)
    else:
        builder, frames = DLA34CenterNet, 4
        video = moving_rectangles_video(frames=frames, height=544, width=960, n_rect=12, min_size=30,
                                        max_size=200, min_speed=1, max_speed=5)
    small = moving_rectangles_video(frames=2, height=64, width=96, n_rect=2, min_size=8, max_size=24)
    ref, dut = _build(builder, torch.float16, 0.05, _calibrated(builder, small))
    n = run_teacher_forced(ref, dut, video, torch.float16)
    assert n % frames == 0 and n // frames >= (400 if network == "hrnet_w32" else 150), n
