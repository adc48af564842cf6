"""Exactness at the layer widths of real models of the family, not only at the
tiny ones: a few layers of the Qwen2.5 0.5B, 1.5B, 3B, 7B and 32B sizes (hidden width,
heads, head size, feed-forward width as in those models' config.json) with
random weights, an 80-token request run whole, most of it at once with the
last 32 tokens one by one, and in portions, in float32 (the reference's 1e-5
criterion, tests/unit/test_layer0_parity.mojo:46 there) and in bfloat16,
against the plain implementation.

The 0.5B case keeps the full vocabulary of 151,936 rows; the others
cut it to a few thousand rows (a count that is no multiple of anything) and
keep one layer, so that the plain NumPy side stays within seconds."""
import numpy as np
import pytest

from helpers import assert_close, bulk_and_tail, collect, plain_logits, portions, random_ids, whole

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]

WIDTHS = {
    # name: config.json of the real model's sizes; "real" lists the keys that are the model's own
    "0.5b": dict(num_hidden_layers=2, hidden_size=896, num_attention_heads=14, num_key_value_heads=2, intermediate_size=4864,
                 vocab_size=151936, tie_word_embeddings=True),
    "1.5b": dict(num_hidden_layers=1, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                 vocab_size=3001, tie_word_embeddings=True),
    "3b": dict(num_hidden_layers=1, hidden_size=2048, num_attention_heads=16, num_key_value_heads=2, intermediate_size=11008,
               vocab_size=2999, tie_word_embeddings=True),
    "7b": dict(num_hidden_layers=1, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
               vocab_size=3003, tie_word_embeddings=False),
    "32b": dict(num_hidden_layers=1, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=27648,
                vocab_size=2051, tie_word_embeddings=False),
}
REAL_KEYS = {"0.5b": "hidden_size heads kv_heads head_dim intermediate_size vocab_size tying",
             "1.5b": "hidden_size heads kv_heads head_dim intermediate_size tying", "3b": "hidden_size heads kv_heads head_dim intermediate_size tying",
             "7b": "hidden_size heads kv_heads head_dim intermediate_size tying", "32b": "hidden_size heads kv_heads head_dim intermediate_size tying"}


def config_of(name):
    return dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", rope_theta=1000000.0, rms_norm_eps=1e-6,
                use_sliding_window=False, max_position_embeddings=32768, **WIDTHS[name])


@pytest.fixture(scope="module", params=list(WIDTHS))
def sized(request, tmp_path_factory):
    from alofa_amd.weights import write_random_model
    name = request.param
    d = tmp_path_factory.mktemp(f"widths_{name.replace('.', '_')}")
    print(f"writing {name} widths ({REAL_KEYS[name]} as in the real model)", flush=True)
    write_random_model(config_of(name), d, seed=2000 + len(name))
    ids = random_ids(5, 80, WIDTHS[name]["vocab_size"])
    print(f"plain model at {name} widths", flush=True)
    ref = plain_logits(d, tuple(ids))
    return name, d, ids, ref


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_at_real_widths(sized, dtype):
    from alofa_amd.replay import Replayer
    from helpers import plain_model
    name, d, ids, ref = sized
    print(f"{name} {dtype}", flush=True)
    r = Replayer(d, dtype, 256)
    got = collect(r, whole("w", ids))["w"]
    assert_close(got, ref, dtype, f"{name} whole")
    if dtype == "float32":
        rel = float(np.abs(got.astype(np.float64) - ref).max() / max(1.0, np.abs(ref).max()))
        print(f"{name} float32 whole: max abs diff / max(1, max|ref|) = {rel:.2e}", flush=True)
    tail = collect(r, bulk_and_tail("t", ids))["t"]
    assert_close(tail, ref, dtype, f"{name} bulk+tail")
    cut = collect(r, portions("p", ids))["p"]
    assert_close(cut, ref, dtype, f"{name} portions")
    if dtype == "float32":      # the cutting changes nothing beyond rounding
        scale = max(1.0, float(np.abs(ref).max()))
        assert np.abs(tail - got).max() <= 2e-6 * scale and np.abs(cut - got).max() <= 2e-6 * scale
    else:
        assert (got.argmax(1) == ref.argmax(1)).mean() >= 0.9
    r.cache.check()
    if dtype == "bfloat16":     # the last use of this size: let the plain side's weights go
        plain_model.cache_clear()


def test_six_layers_of_the_half_billion_model_against_the_librarys_own_plain_path(tmp_path):
    """The library's plain path (C++ on the host: float64 sums in formula order, contiguous keys and values; the NumPy
    transcription in tests/plain pins it on the tiny models) as a second twin where NumPy would take minutes: six
    layers of the 0.5B widths with the full vocabulary, 96 tokens, float32 at the reference's 1e-5 in two cuttings."""
    from alofa_amd.plain import PlainModel
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    cfg = dict(config_of("0.5b"), num_hidden_layers=6)
    write_random_model(cfg, tmp_path, seed=2100)
    ids = random_ids(6, 96, cfg["vocab_size"])
    print("the library's plain path, six layers at 0.5B widths", flush=True)
    ref = PlainModel(tmp_path, max_tokens=128).run(ids)
    r = Replayer(tmp_path, "float32", 256)
    assert_close(collect(r, whole("w", ids))["w"], ref, "float32", "six layers whole")
    assert_close(collect(r, bulk_and_tail("t", ids))["t"], ref, "float32", "six layers bulk+tail")
