"""Backend calls recorded into a HIP graph and replayed (``tannic_hip_graph_*``, ``tannic_amd.Graph``).

A replay must give what the eager calls give, every time: the graph is launched several times with the program's own
eager work and waits between the launches, and each replay is compared bit for bit with the eager result."""
import ctypes as C

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import abi, decoder_layer as dl, ops

pytestmark = pytest.mark.gpu


def small_layer(dtype, env, seed):
    s = dl.LayerShape(hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512)
    seq = 48
    w = {}
    for i, (name, shape) in enumerate(dl.weight_shapes(s).items()):
        values = np.ones(shape) if name.startswith("g") else support.normal(seed, 10 + i, shape, 0.05)
        w[name] = ta.tensor(values, dtype, env)
    x = ta.tensor(support.normal(seed, 1, (1, seq, s.hidden), 1.0), dtype, env)
    cos, sin = dl.rotary_tables(s, seq, dtype, env)
    return s, w, x, cos, sin, dl.causal_mask(seq, dtype, env), ta.tensor(np.ones(1), dtype, env)


def eager_noise(env, rounds=3):
    """Eager work of the sizes the layer uses: takes and returns blocks the way an unrelated caller would."""
    kept = []
    for r in range(rounds):
        a = ta.tensor(support.normal(50 + r, 0, (1, 48, 256), 1.0), ta.bfloat16, env)
        b = ops.add(a, a)
        c = ops.matmul(b, ta.tensor(support.normal(60 + r, 0, (256, 512), 0.1), ta.bfloat16, env))
        kept.append((ops.mul(c, c), None))
    return kept


@pytest.mark.parametrize("dtype", [ta.bfloat16, ta.float32], ids=["bfloat16", "float32"])
def test_replays_of_a_layer_equal_the_eager_layer(device, dtype):
    s, w, x, cos, sin, mask, one = small_layer(dtype, device, 5)
    want = dl.forward(s, w, x, cos, sin, mask, one).storage()
    with ta.Graph(device) as g:
        y = dl.forward(s, w, x, cos, sin, mask, one)
    for replay in range(4):
        g.launch()
        np.testing.assert_array_equal(y.storage(), want, err_msg=f"replay {replay}")
        eager_noise(device)
        # the eager layer between replays gives the same too (it shares the stream and the kept blocks with the graph)
        np.testing.assert_array_equal(dl.forward(s, w, x, cos, sin, mask, one).storage(), want)
    g.close()
    np.testing.assert_array_equal(y.storage(), want)      # a live tensor outlives the recording that made it


def test_replay_reads_the_inputs_as_they_are_at_launch(device):
    s, w, x, cos, sin, mask, one = small_layer(ta.bfloat16, device, 6)
    with ta.Graph(device) as g:
        y = dl.forward(s, w, x, cos, sin, mask, one)
    g.launch()
    first = y.storage()
    other = ta.tensor(support.normal(7, 1, x.shape, 1.0), ta.bfloat16, device)
    want = dl.forward(s, w, other, cos, sin, mask, one).storage()
    ops.copy_into(x, other)
    g.launch()
    second = y.storage()
    np.testing.assert_array_equal(second, want)
    assert (first != second).any()


def test_a_recording_keeps_its_memory_to_itself(device):
    """Tensors allocated after the recording, of the sizes of its temporaries, are not written by a replay."""
    s, w, x, cos, sin, mask, one = small_layer(ta.bfloat16, device, 8)
    with ta.Graph(device) as g:
        y = dl.forward(s, w, x, cos, sin, mask, one)
    g.launch()
    want = y.storage()
    sizes = [(1, 48, 256), (1, 48, 512), (1, 4, 48, 48), (1, 4, 48, 64), (1, 2, 48, 64), (48, 64)]
    bystanders = []
    for i, shape in enumerate(sizes * 6):
        values = support.normal(9, i, shape, 1.0)
        t = ta.tensor(values, ta.bfloat16, device)
        bystanders.append((t, t.storage()))
    g.launch()
    g.launch()
    np.testing.assert_array_equal(y.storage(), want)
    for t, before in bystanders:
        np.testing.assert_array_equal(t.storage(), before)


def test_products_that_share_k_replay_with_their_partial_sums(device):
    """A product whose workgroups share K keeps partial sums in library scratch; eager products use scratch between replays."""
    a = ta.tensor(support.normal(11, 0, (128, 4096), 1.0), ta.float16, device)
    b = ta.tensor(support.normal(11, 1, (4096, 4096), 0.02), ta.float16, device)
    c = ta.tensor(support.normal(11, 2, (96, 2048), 1.0), ta.float16, device)
    d = ta.tensor(support.normal(11, 3, (1024, 2048), 0.02), ta.float16, device)
    want = ops.matmul(a, b.transpose()).storage()
    with ta.Graph(device) as g:
        y = ops.matmul(a, b.transpose())
        z = ops.add(y, y)
    for replay in range(3):
        g.launch()
        np.testing.assert_array_equal(y.storage(), want, err_msg=f"replay {replay}")
        ops.matmul(c, d.transpose())
        ops.matmul(a, b.transpose())
    assert z.shape == y.shape


def test_every_operator_family_replays(device):
    """One recording that holds kernels of every family, those with library scratch among them (the gathered signal of
    an fp32 convolution, the rearranged weights of a 16-bit one, partial results of a column reduction, partial sums of
    a product): two replays with other eager work in between equal the eager results bit for bit."""
    f16, f32 = ta.float16, ta.float32
    img16 = ta.tensor(support.normal(13, 0, (4, 64, 28, 28), 1.0), f16, device)
    ker16 = ta.tensor(support.normal(13, 1, (64, 64, 3, 3), 0.05), f16, device)
    img32 = ta.tensor(support.normal(13, 2, (2, 6, 20, 20), 1.0), f32, device)
    ker32 = ta.tensor(support.normal(13, 3, (5, 6, 3, 3), 0.3), f32, device)
    bias32 = ta.tensor(support.normal(13, 4, (5,), 1.0), f32, device)
    big = ta.tensor(support.normal(13, 5, (16, 2048, 96), 1.0), f32, device)
    other = ta.tensor(support.normal(13, 6, (16, 2048, 96), 1.0), f32, device)
    rows = ta.tensor(support.normal(13, 7, (300, 1000), 1.0), ta.bfloat16, device)
    gain = ta.tensor(support.normal(13, 8, (1000,), 1.0), ta.bfloat16, device)
    a = ta.tensor(support.normal(13, 9, (96, 4096), 1.0), f16, device)
    b = ta.tensor(support.normal(13, 10, (2048, 4096), 0.02), f16, device)
    rho = ta.tensor(support.uniform(13, 11, (40, 30), 0.5, 2.0), f32, device)
    theta = ta.tensor(support.uniform(13, 12, (40, 30), -3.0, 3.0), f32, device)
    # operands that are copied into aligned rows first (an odd number of columns), a matrix times a column, a handful of
    # very long rows shared by several blocks, a transposing copy, the unfolded batch of a convolution
    odd_a = ta.tensor(support.normal(13, 13, (300, 1032), 1.0), f16, device)
    odd_b = ta.tensor(support.normal(13, 14, (1032, 1001), 0.05), f16, device)
    column = ta.tensor(support.normal(13, 15, (4096, 1), 0.05), f16, device)
    logits = ta.tensor(support.normal(13, 16, (4, 50257), 2.0), f32, device)
    img7 = ta.tensor(support.normal(13, 17, (8, 128, 7, 7), 1.0), f16, device)
    ker7 = ta.tensor(support.normal(13, 18, (64, 128, 3, 3), 0.05), f16, device)

    # products that convert an operand of another type first, float64 on its matrix kernel, a float64 convolution through
    # the unfolded batch, a few fp32 rows times a row-major matrix (partial sums of workgroups that share K), int8 few rows
    wide32 = ta.tensor(support.normal(13, 19, (200, 1024), 1.0), f32, device)
    w_bf16 = ta.tensor(support.normal(13, 20, (512, 1024), 0.05), ta.bfloat16, device)
    a64 = ta.tensor(support.normal(13, 21, (300, 260), 1.0), ta.float64, device)
    b64 = ta.tensor(support.normal(13, 22, (260, 200), 1.0), ta.float64, device)
    img64 = ta.tensor(support.normal(13, 23, (2, 8, 12, 12), 1.0), ta.float64, device)
    ker64 = ta.tensor(support.normal(13, 24, (16, 8, 3, 3), 0.3), ta.float64, device)
    few32 = ta.tensor(support.normal(13, 25, (3, 2048), 1.0), f32, device)
    w32 = ta.tensor(support.normal(13, 26, (2048, 1024), 0.05), f32, device)
    few8 = ta.tensor(support.integers(13, 27, (4, 512), -100, 100), ta.int8, device)
    w8 = ta.tensor(support.integers(13, 28, (640, 512), -100, 100), ta.int8, device)

    def everything():
        return [
            ops.matmul(wide32, w_bf16.transpose()), ops.matmul(a64, b64), ops.convolve2d(img64, ker64, None, 1, 1),
            ops.matmul(few32, w32), ops.matmul(few8, w8.transpose()),
            ops.convolve2d(img16, ker16, None, 1, 1),
            ops.convolve2d(img32, ker32, bias32, 2, 1),
            ops.sum(big, 1), ops.mean(big, 0), ops.argmax(big, 1), ops.max(big, 2),
            ops.gt(big, other), ops.add(ops.exp(ops.neg(ops.abs(big))), other),
            ops.realify(ops.polar(rho, theta)),
            ops.repeat(img32, 3, 1), ops.concatenate(big, other, 2), ops.triu(rho, 1), ops.outer(bias32, bias32),
            ops.softmax(rows), ops.rms_norm(rows, gain), ops.cast(rows, f32),
            ops.matmul(a, b.transpose()),
            ops.matmul(odd_a, odd_b), ops.matmul(b, column), ops.argmax(logits, 1), ops.softmax(logits), ops.sum(logits, 1),
            ops.repack(b.transpose()), ops.convolve2d(img7, ker7, None, 1, 1),
        ]

    want = [t.storage() for t in everything()]
    with ta.Graph(device) as g:
        recorded = everything()
    for replay in range(2):
        g.launch()
        for i, (t, w) in enumerate(zip(recorded, want)):
            np.testing.assert_array_equal(t.storage(), w, err_msg=f"replay {replay}, result {i}")
        for t, w in zip(everything(), want):       # eager calls take the same scratch between replays
            np.testing.assert_array_equal(t.storage(), w)
        eager_noise(device)


def test_the_product_that_allocates_nothing_can_be_recorded(device):
    """tannic_hip_gemm_noalloc with a destination that exists before the recording: the recording holds kernels only
    (the partial sums of the shared K live in the library's static array), and replays equal tannic_hip_gemm."""
    a = ta.tensor(support.normal(12, 0, (128, 4096), 1.0), ta.float16, device)
    b = ta.tensor(support.normal(12, 1, (4096, 4096), 0.02), ta.float16, device).transpose()
    want = ops.matmul(a, b).storage()
    dst = ta.Tensor(ta.float16, (128, 4096)).initialize(device)
    lib = ta.library()
    with ta.Graph(device) as g:
        status = lib.kernels["gemm_noalloc"](a.reference(), b.reference(), dst.reference(), device.stream())
        assert status == abi.SUCCESS, lib.error_message()
    for replay in range(3):
        ops.copy_into(dst, ta.tensor(np.zeros((128, 4096)), ta.float16, device))
        g.launch()
        np.testing.assert_array_equal(dst.storage(), want, err_msg=f"replay {replay}")
        ops.matmul(a, b)


def test_calls_that_wait_are_refused_while_recording(device):
    x = ta.tensor(np.arange(8.0), ta.float32, device)
    with pytest.raises(ta.BackendError, match="being recorded"):
        with ta.Graph(device):
            y = ops.add(x, x)
            y.numpy()
    # the failed recording is gone; the device works as before
    np.testing.assert_array_equal(ops.add(x, x).numpy(), 2 * np.arange(8.0))
    with ta.Graph(device) as g:
        y = ops.add(x, x)
    g.launch()
    np.testing.assert_array_equal(y.numpy(), 2 * np.arange(8.0))
    with pytest.raises(ta.BackendError):
        with ta.Graph(device):
            with ta.Graph(device):
                pass
    np.testing.assert_array_equal(ops.add(x, x).numpy(), 2 * np.arange(8.0))
