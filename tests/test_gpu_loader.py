"""A model read from the reference's parameter files gives the same hidden states, logits, tokens and cache bytes as
the model built from the arrays those files were written from (real hidden sizes, one layer, small vocabulary so the files stay at ~65 MB)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_loaded_model_equals_source_model(tmp_path):
    import flexllm_amd as fx
    from flexllm_amd import llama, loader
    cfg = llama.make_config(layers=1, vocab=512, max_pos=256)
    host_w = llama.synth_weights(cfg, seed=11, device=False)
    d = str(tmp_path / "parameters")
    loader.save_reference_parameters(d, cfg, host_w)
    loaded = loader.load_reference_parameters(d, cfg, device=True)
    assert np.array_equal(loaded["wg"][0].numpy(), host_w["wg"][0])
    assert np.array_equal(loaded["embed"].numpy().view(np.uint16), host_w["embed"])
    src = llama.synth_weights(cfg, seed=11, device=True)
    from flexllm_amd import synth
    outs = []
    for w in (loaded, src):
        model = llama.Llama(cfg, w)
        got = []
        for pos in range(3):
            x = synth.host_normal_f32((cfg["hidden"],), 900 + pos)
            hid, logits = model.decode_hidden(fx.to_device(x), pos, want_logits=True)
            got += [hid.numpy().copy(), logits.numpy().copy()]
        tok = fx.to_device(np.array([77], np.int32))
        out = fx.zeros((4,), np.int32)
        model.decode_greedy(tok, 3, 4, out, use_graph=False)    # exercises the embedding table
        got.append(out.numpy().copy())
        model.check()
        k, v = model.caches_token_major()
        got += [k.copy(), v.copy()]
        outs.append(got)
        model.close()
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
    assert np.abs(outs[0][1]).max() > 0 and outs[0][-2].any()


def test_loaded_w4a4_model_equals_source_model(tmp_path):
    """The same for the W4A4 configuration: files with int4 values, row sums and the int4 head -> the W4A4 model."""
    import flexllm_amd as fx
    from flexllm_amd import llama, loader, synth
    cfg = llama.make_config(layers=1, vocab=512, max_pos=256)
    host_w = llama.synth_weights_w4a4(cfg, seed=12, device=False, embed_range=0.05)
    d = str(tmp_path / "parameters")
    loader.save_reference_parameters(d, cfg, host_w)
    loaded = loader.load_reference_parameters(d, cfg, device=True, w4a4=True)
    src = {k: ([fx.to_device(a) for a in v] if isinstance(v, list) else
               fx.to_device(v.view(np.float16) if k == "embed" else v)) for k, v in host_w.items()}
    outs = []
    for w in (loaded, src):
        model = llama.Llama(cfg, w)
        assert model.w4a4
        got = []
        for pos in range(2):
            x = synth.host_normal_f32((cfg["hidden"],), 910 + pos)
            hid, logits = model.decode_hidden(fx.to_device(x), pos, want_logits=True)
            got += [hid.numpy().copy(), logits.numpy().copy()]
        got.append(np.array(model.generate(np.arange(5, 38, dtype=np.int32), 4)))      # prefill of 32 tokens + 4 greedy ones
        model.check()
        k, v = model.caches_token_major()
        got += [k.copy(), v.copy()]
        outs.append(got)
        model.close()
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
    assert np.abs(outs[0][1]).max() > 0 and outs[0][-2].any()
