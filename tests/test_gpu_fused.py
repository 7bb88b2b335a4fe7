"""GPU: the one-kernel decode step (tg_set_fused_decode; tiny-gemma_amd/csrc/tg_decode_fused.hip) against the launch
path.  Both paths run the same per-column arithmetic in the same order (the device code is shared), so everything
must be bit-identical: greedy ids, the residual stream after every block, logits and every KV-cache slot.

The fused step is opt-in (it is slower than one launch per projection on this machine); these tests keep it honest.
Its waits between workgroups are bounded: the last test forces the bound from the host (one poll per wait), checks
that the kernel still ends, that the error is reported and that the session continues on the launch path."""
import numpy as np
import pytest

import golden_inputs as gi

pytestmark = pytest.mark.gpu


def make(tg, weight_images, name):
    shape, n_layers, seed, n_prompt, nd, nt, gsize = gi.MODEL_CASES[name]
    model = tg.Transformer(tg.named_config(shape, n_layers))
    model.read_weights_mem(weight_images(shape, n_layers, seed))
    return model, gi.prompt_ids(seed, n_prompt), gsize, n_layers


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def stepwise(tg, model, prompt, gsize, n_layers, fused, n_steps):
    tg.lib().tg_set_fused_decode(fused, 0, 1 << 18)
    sess = model.session(gsize=gsize)
    tok, _ = sess.prefill(prompt)
    out = []
    for _ in range(n_steps):
        tok, logits = sess.decode(tok)
        out.append((tok, bits(logits).copy(), bits(sess.taps(rows=1)).copy()))
    kv = [sess.kv(l)[:2] for l in range(n_layers)]
    return out, kv


@pytest.mark.parametrize("name,n_steps", [("small6", 12), ("small6_window", 6)])
def test_fused_step_is_bit_identical_to_the_launch_path(tg, weight_images, name, n_steps):
    """270m-shaped 6-layer model (one global layer): a 70-token prompt, and a 600-token prompt whose local layers
    run on the 512-slot ring with the position past the window."""
    model, prompt, gsize, n_layers = make(tg, weight_images, name)
    a, kva = stepwise(tg, model, prompt, gsize, n_layers, 0, n_steps)
    b, kvb = stepwise(tg, model, prompt, gsize, n_layers, 1, n_steps)
    for i, ((ta, la, xa), (tb, lb, xb)) in enumerate(zip(a, b)):
        assert ta == tb, i
        assert np.array_equal(xa, xb), (i, [int((xa[k] != xb[k]).sum()) for k in range(xa.shape[0])])
        assert np.array_equal(la, lb), i
    for l in range(n_layers):
        assert np.array_equal(bits(kva[l][0]), bits(kvb[l][0])) and np.array_equal(bits(kva[l][1]), bits(kvb[l][1])), l


def test_fused_steps_chained_on_the_device(tg, weight_images):
    """A batch of steps without host round trips: the pick of a step is finished by the next step's launch
    (the pending argmax pairs are folded in its prologue), on both paths; 1B-shaped layers would take the other
    kernel instantiation, covered by the full-size test below."""
    model, prompt, gsize, n_layers = make(tg, weight_images, "small6")
    ids = []
    for fused in (0, 1):
        tg.lib().tg_set_fused_decode(fused, 0, 1 << 18)
        sess = model.session(gsize=gsize)
        sess.prefill(prompt)
        sess.decode_enqueue(40)
        ids.append(sess.read_ids(64))
    assert ids[0].size == 41 and np.array_equal(ids[0], ids[1])


def test_fused_step_1B_shape(tg, weight_images):
    """The 1B shape (26 layers; the instantiation with 9 and 7 register steps per tile), 178-token prompt."""
    model, prompt, gsize, n_layers = make(tg, weight_images, "full1B")
    a, kva = stepwise(tg, model, prompt, gsize, n_layers, 0, 3)
    b, kvb = stepwise(tg, model, prompt, gsize, n_layers, 1, 3)
    for i, ((ta, la, xa), (tb, lb, xb)) in enumerate(zip(a, b)):
        assert ta == tb and np.array_equal(xa, xb) and np.array_equal(la, lb), i
    for l in (0, 5, 25):
        assert np.array_equal(bits(kva[l][0]), bits(kvb[l][0])) and np.array_equal(bits(kva[l][1]), bits(kvb[l][1])), l


def test_fused_step_gives_up_cleanly(tg, weight_images):
    """max_spins = 1: every wait between workgroups gives up after one poll.  The kernel must still end, the next
    read-back must report TG_ERR_STATE, and after a reset the session must produce the launch path's ids."""
    model, prompt, gsize, n_layers = make(tg, weight_images, "small6")
    tg.lib().tg_set_fused_decode(0, 0, 0)
    ref = model.session(gsize=gsize)
    ref.prefill(prompt)
    ref.decode_enqueue(8)
    want = ref.read_ids(16)
    tg.lib().tg_set_fused_decode(1, 0, 1)
    sess = model.session(gsize=gsize)
    sess.prefill(prompt)
    sess.decode_enqueue(2)
    with pytest.raises(tg.TgError) as e:
        sess.read_ids(16)
    assert e.value.code == -7 and "bounded wait" in str(e.value)  # TG_ERR_STATE
    sess.reset()
    sess.prefill(prompt)
    sess.decode_enqueue(8)          # the knob is still on: the session itself has left the fused path
    assert np.array_equal(sess.read_ids(16), want)
