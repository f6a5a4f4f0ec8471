"""Host-side contract: executor registration, module surgery, planning, state dicts, plugins.

Restates the properties the reference's own tests pin for this path --
thunder/tests/test_extend.py:23-302 (executor API), thunder/tests/test_transforms.py:116-230,
293-344 (quantisation on real / meta modules, tied weights, materialisation), and the disabled
thunder/tests/test_networks.py:284-357 (state-dict round trips).

Every test runs twice: on the CPU with tests/fake_backend.py standing in for the kernels (host
logic only), and, marked ``gpu``, against libnf4hip.so on the MI355X.
"""

import pytest
import torch
from torch.testing import assert_close

import fake_backend

BACKENDS = [pytest.param("fake-cpu", id="cpu"), pytest.param("hip", marks=pytest.mark.gpu, id="hip")]


@pytest.fixture(params=BACKENDS)
def dev(request, ta, oracle):
    if request.param == "hip":
        yield "cuda"
    else:
        with fake_backend.installed(ta):
            yield "cpu"


# ---- executor API -----------------------------------------------------------------------------------


def test_executor_api(ta):
    ex = ta.extend.OperatorExecutor("myex", version=0.3)
    assert ex.name == "myex" and ex.version == 0.3
    assert ex == ta.extend.OperatorExecutor("myex") and hash(ex) == hash("myex")  # identity is the name

    def meta(a, b):
        return ta.TensorProxy(like=a)

    with pytest.raises(AssertionError, match="neither was"):
        ex.register_operator("f")
    with pytest.raises(AssertionError, match="both were"):
        ex.register_operator("f", like=ta.extend.linear, meta=meta)
    sym = ex.register_operator("myadd", meta=meta, fn=lambda a, b: a + b)
    assert sym.executor is ex and sym.is_prim and ex.opmap["myadd"] is sym
    bsym = sym.bind(torch.ones(2), torch.ones(2))
    assert bsym._call_ctx == {"myadd": bsym._call_ctx["myadd"]} and bsym.sym.executor is ex
    assert_close(sym(torch.ones(2), torch.ones(2)), torch.full((2,), 2.0))
    p = sym(ta.TensorProxy("a", shape=(2, 3), dtype=torch.float32, device="cpu"), None)
    assert isinstance(p, ta.TensorProxy) and p.shape == (2, 3)
    like = ex.register_operator("mylinear", like=ta.extend.linear, fn=torch.nn.functional.linear)
    assert not like.is_prim and like.meta is ta.extend.linear

    ex.register_implementation(ta.extend.linear, like, checker=lambda a, w, b=None: a.dtype == torch.float32)
    b32 = ta.extend.linear.bind(torch.ones(1, 2), torch.ones(2, 2), None)
    b16 = ta.extend.linear.bind(torch.ones(1, 2, dtype=torch.bfloat16), torch.ones(2, 2), None)
    assert ex.can_execute(b32) and not ex.can_execute(b16) and not ex.can_execute(bsym)

    assert ta.extend.get_executor("myex") is None
    ta.extend.register_executor(ex)
    try:
        assert ta.extend.get_executor("myex") is ex and ex in ta.extend.get_all_executors()
        assert ta.extend.resolve_executors(["myex", ex]) == (ex, ex)
        with pytest.raises(ValueError, match="nosuch"):
            ta.extend.resolve_executors(["nosuch"])
        with pytest.raises(ValueError, match="neither an Executor nor the name of one"):
            ta.extend.resolve_executors([3])
        ta.extend.add_default_executor(ex)
        assert ta.extend.get_default_executors()[0] is ex and ta.extend.resolve_executors(None)[0] is ex
        assert ta.extend.add_executor_lists([ex], ["myex"]) == [ex]
    finally:
        ta.extend.deregister_executor(ex)
    assert ta.extend.get_executor("myex") is None and ex not in ta.extend.get_default_executors()

    sx = ta.extend.single_op_executor("oneop", "mul2", lambda a: a * 2, lambda a: ta.TensorProxy(like=a))
    try:
        assert ta.extend.get_executor("oneop") is sx and sx.opmap["mul2"].executor is sx
        assert sx.can_execute(sx.opmap["mul2"].bind(torch.ones(1)))
    finally:
        ta.extend.deregister_executor(sx)


def test_nf4_executor_is_a_singleton_with_the_reference_signature(ta):
    ex = ta.get_hip_nf4_executor()
    assert ex is ta.get_hip_nf4_executor() is ta.get_bitsandbytes_executor()
    assert ex.name == "quant_hip_nf4" and ta.extend.get_executor("quant_hip_nf4") is ex
    op = ex.opmap["hip_matmul_nf4"]
    assert op.executor is ex and set(ex.opmap) == {"hip_matmul_nf4", "hip_quantize_nf4", "hip_dequantize_nf4",
                                                   "hip_matmul_nf4_dq", "hip_quantize_nf4_dq", "hip_dequantize_nf4_dq",
                                                   "hip_matmul_nf4_epilogue"}
    x = ta.TensorProxy("x", shape=(2, 3, 64), dtype=torch.bfloat16, device="cpu")
    out = op(x, None, None, None, None, 64, torch.bfloat16, (128, 64))
    assert out.shape == (2, 3, 128) and out.dtype == torch.bfloat16 and out.device == x.device
    with pytest.raises(AssertionError):
        op(x, None, None, None, None, 64, torch.bfloat16, (128, 32))  # K mismatch
    with pytest.raises(AssertionError):
        op(x, None, None, None, None, 64, torch.bfloat16, (128,))
    qw, absmax, code = ex.opmap["hip_quantize_nf4"](ta.TensorProxy("w", shape=(3, 21), dtype=torch.float16, device="cpu"))
    assert qw.shape == (32, 1) and qw.dtype == torch.uint8 and absmax.shape == (1,) and code.shape == (16,)
    # the double-quant siblings: tensors in place of absmax, nested_blocksize after blocksize
    w = ta.TensorProxy("w", shape=(1024, 512), dtype=torch.bfloat16, device="cpu")
    qw, aq, a2, m256, off, code = ex.opmap["hip_quantize_nf4_dq"](w)
    assert (qw.shape, aq.shape, a2.shape, m256.shape, off.shape, code.shape) == ((262144, 1), (8192,), (32,), (256,), (1,), (16,))
    assert aq.dtype == torch.uint8 and a2.dtype == m256.dtype == off.dtype == torch.float32
    out = ex.opmap["hip_matmul_nf4_dq"](x, None, None, None, None, None, None, None, 64, 256, torch.bfloat16, (128, 64))
    assert out.shape == (2, 3, 128) and out.dtype == torch.bfloat16
    with pytest.raises(AssertionError):
        ex.opmap["hip_matmul_nf4_dq"](x, None, None, None, None, None, None, None, 64, 256, torch.bfloat16, (128, 32))
    deq = ex.opmap["hip_dequantize_nf4_dq"](qw, aq, a2, m256, off, code, 64, 256, torch.bfloat16, (1024, 512))
    assert deq.shape == (1024, 512) and deq.dtype == torch.bfloat16


def test_plugin_registry(ta):
    assert ta.get_plugin("quantize-int4") is ta.QuantizeInt4 and "quantize-int4" in ta.get_plugin_names()
    p = ta.QuantizeInt4()
    assert p.policy is ta.PluginPolicy.PRE and p.setup_lookasides() is None
    (t,) = p.setup_transforms()
    assert isinstance(t, ta.BitsAndBytesLinearQuant4bit) and p.setup_executors() == [ta.get_hip_nf4_executor()]

    class Mine(ta.Plugin):
        pass

    ta.register_plugin("mine", Mine)
    assert ta.get_plugin("mine") is Mine
    del ta.plugins.names_to_plugins["mine"]
    with pytest.raises(ValueError, match="not recognized"):
        ta.compile(torch.nn.Linear(2, 2), plugins="no-such-plugin")
    with pytest.raises(NotImplementedError):
        ta.jit(lambda x: x)


# ---- the transform --------------------------------------------------------------------------------


def _mlp(dev, dtype=torch.float32):
    torch.manual_seed(42)
    with torch.device(dev):
        m = torch.nn.Sequential(torch.nn.Linear(512, 1024), torch.nn.GELU(), torch.nn.Linear(1024, 512))
    return m.to(dtype).eval().requires_grad_(False)


def test_quantized_mlp_matches_eager_and_plan_metadata(ta, dev):
    """thunder/tests/test_transforms.py:189-230 (fp32 MLP with bias, x [1, 512]): quantised vs
    unquantised within 2e-1, and every computation input's shape/device/dtype equals both the
    runtime tensor and the prologue's output proxy."""
    mlp = _mlp(dev)
    inp = torch.randn(1, 512, device=dev)
    jm = ta.jit(mlp, executors=(ta.get_hip_nf4_executor(),), transforms=[ta.BitsAndBytesLinearQuant4bit()])
    assert isinstance(jm, ta.ThunderModule)
    actual, expected = jm(inp), mlp(inp)
    assert_close(actual, expected, atol=2e-1, rtol=2e-1)
    assert not torch.equal(actual, expected)
    comp, pro = ta.last_traces(jm)[-1], ta.last_prologue_traces(jm)[-1]
    names = ["0.weight", "0.bias", "2.weight", "2.bias", "0.weight.absmax", "0.weight.code", "2.weight.absmax", "2.weight.code"]
    assert [a.name for a in comp.args] == ["t_" + n.replace(".", "_") for n in names]
    assert len(comp.args) == len(pro.output[0])
    for n, cproxy, pproxy in zip(names, comp.args, pro.output[0]):
        t = jm.get_parameter(n)
        assert cproxy.shape == pproxy.shape == tuple(t.shape)
        assert cproxy.dtype == pproxy.dtype == t.dtype
        assert cproxy.device.type == pproxy.device.type == t.device.type
    calls = [b for b in comp.bound_symbols if b.sym.name == "hip_matmul_nf4"]
    assert len(calls) == 2 and all(b.sym.executor is ta.get_hip_nf4_executor() for b in calls)
    assert not [b for b in comp.bound_symbols if b.sym is ta.extend.linear]
    b0 = calls[0]
    assert [getattr(a, "name", a) for a in b0.args] == ["t_0_input", "t_0_weight", "t_0_bias", "t_0_weight_absmax",
                                                        "t_0_weight_code", 64, torch.float32, (1024, 512)]
    assert "STATIC_MEMORY_LOCATION" in b0.args[3].tags and "STATIC_MEMORY_LOCATION" in b0.args[4].tags
    # the user's module is untouched
    assert mlp[0].weight.dtype == torch.float32 and mlp[0].weight.shape == (1024, 512)


def test_quant_states_and_overrides(ta, dev, oracle):
    mlp = _mlp(dev, torch.bfloat16)
    tr = ta.BitsAndBytesLinearQuant4bit()
    jm = ta.jit(mlp, transforms=[tr], executors=(ta.get_hip_nf4_executor(),))
    assert tr.quantized_submodule_names == {"0", "2"} and set(tr.quant_states) == {"0.weight", "2.weight"}
    qs = tr.quant_states["0.weight"]
    assert qs == {"dtype": torch.bfloat16, "shape": (1024, 512), "blocksize": 64, "qweight.dtype": torch.uint8,
                  "qweight.shape": (262144, 1), "absmax.dtype": torch.float32, "absmax.shape": (8192,),
                  "code.dtype": torch.float32, "code.shape": (16,), "device": mlp[0].weight.device}
    qw, absmax = oracle.C().quantize(mlp[0].weight, 64)
    assert torch.equal(jm.get_parameter("0.weight").cpu(), qw)
    assert torch.equal(jm.get_parameter("0.weight.absmax").cpu(), absmax)
    assert torch.equal(jm.get_parameter("0.weight.code").cpu(), oracle.nf4_lut())
    assert not isinstance(jm.get_parameter("0.weight"), torch.nn.Parameter)
    sd = jm.state_dict()
    assert list(sd) == ["0.weight", "0.bias", "2.weight", "2.bias", "0.weight.absmax", "0.weight.code",
                        "2.weight.absmax", "2.weight.code"]
    assert sd["0.weight"].dtype == torch.uint8 and sd["0.weight"].shape == (262144, 1)
    assert dict(jm.named_parameters())["2.weight.absmax"].shape == (8192,)
    assert jm.training is False and jm._model[0] is mlp[0] and jm.get_submodule("0") is mlp[0]  # attributes fall through


def test_tied_weights_and_materialization_from_module_init(ta, dev):
    """thunder/tests/test_transforms.py:293-344: Linear(2,2) x3 with 0.weight tied to 4.weight (n = 4,
    one partial block); a meta model materialised with the module's own init under the same seed
    equals direct quantisation."""

    def get_model():
        m0 = torch.nn.Linear(2, 2)
        with torch.device("meta"):
            m4 = torch.nn.Linear(2, 2)
        m4.weight, m4.bias = m0.weight, m0.bias
        return torch.nn.Sequential(m0, torch.nn.GELU(), torch.nn.Linear(2, 2), torch.nn.GELU(), m4).eval().requires_grad_(False)

    ex = ta.get_hip_nf4_executor()
    torch.manual_seed(1234)
    with torch.device(dev):
        m_ref = get_model()
        inp = torch.randn(3, 2)
    jm_ref = ta.jit(m_ref, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=(ex,))
    torch.manual_seed(1234)
    with torch.device("meta"):
        m = get_model()
    jm = ta.jit(m, executors=(ex,), transforms=[
        ta.BitsAndBytesLinearQuant4bit(),
        ta.MaterializationTransform(dev, init=ta.MaterializationTransform.init_from_original_module_init())])
    assert_close(jm(inp), jm_ref(inp))
    assert jm_ref._get_shared_names()["0.weight"] == {"0.weight", "4.weight"}
    assert jm._get_shared_names()["0.weight"] == {"0.weight", "4.weight"}
    for j in (jm, jm_ref):
        for suffix in ("", ".absmax", ".code"):
            assert j.get_parameter("0.weight" + suffix) is j.get_parameter("4.weight" + suffix)
        assert j.get_parameter("0.weight").shape == (2, 1) and j.get_parameter("0.weight.absmax").shape == (1,)
    for n, p in jm_ref.named_parameters():
        assert_close(jm.get_parameter(n), p)
        assert jm.get_parameter(n).device.type == torch.device(dev).type
    # the reference output, for a sanity bound against the unquantised module
    assert_close(jm_ref(inp), m_ref(inp), atol=3e-1, rtol=3e-1)


class TinyLlama(torch.nn.Module):
    """A llama2-like block stack small enough for the CPU: n_embd 64, intermediate 1376 (not a
    multiple of 64, so NF4 blocks straddle weight rows, as in the reference's test model,
    thunder/tests/litgpt_model.py:39-52), a KV cache buffer and a non-persistent rope table."""

    def __init__(self, n_layer=2, n_embd=64, inter=1376, vocab=320, n_head=4, max_seq=16):
        super().__init__()
        self.n_head, self.hd = n_head, n_embd // n_head
        self.wte = torch.nn.Embedding(vocab, n_embd)
        self.layers = torch.nn.ModuleList()
        for _ in range(n_layer):
            blk = torch.nn.Module()
            blk.norm1 = torch.nn.LayerNorm(n_embd)
            blk.qkv = torch.nn.Linear(n_embd, 3 * n_embd, bias=False)
            blk.proj = torch.nn.Linear(n_embd, n_embd, bias=False)
            blk.norm2 = torch.nn.LayerNorm(n_embd)
            blk.fc1 = torch.nn.Linear(n_embd, inter, bias=False)
            blk.fc2 = torch.nn.Linear(n_embd, inter, bias=False)
            blk.down = torch.nn.Linear(inter, n_embd, bias=False)
            blk.register_buffer("k_cache", torch.zeros(1, n_head, max_seq, self.hd))
            blk.register_buffer("v_cache", torch.zeros(1, n_head, max_seq, self.hd))
            self.layers.append(blk)
        self.ln_f = torch.nn.LayerNorm(n_embd)
        self.lm_head = torch.nn.Linear(n_embd, vocab, bias=False)
        self.register_buffer("scale", torch.tensor(self.hd**-0.5), persistent=False)

    def reset_parameters(self):
        with torch.no_grad():
            self.scale.fill_(self.hd**-0.5)

    def forward(self, idx, input_pos):
        x = self.wte(idx)
        B, T, C = x.shape
        for blk in self.layers:
            q, k, v = blk.qkv(blk.norm1(x)).view(B, T, 3, self.n_head, self.hd).permute(2, 0, 3, 1, 4)
            k = blk.k_cache.index_copy_(2, input_pos, k.to(blk.k_cache.dtype))[:, :, : int(input_pos[-1]) + 1]
            v = blk.v_cache.index_copy_(2, input_pos, v.to(blk.v_cache.dtype))[:, :, : int(input_pos[-1]) + 1]
            att = torch.softmax((q @ k.transpose(-1, -2)) * self.scale.to(q.dtype), dim=-1) @ v
            x = x + blk.proj(att.transpose(1, 2).reshape(B, T, C))
            h = blk.norm2(x)
            x = x + blk.down(torch.nn.functional.silu(blk.fc1(h)) * blk.fc2(h))
        return self.lm_head(self.ln_f(x))


def test_quantization_on_meta(ta, dev):
    """thunder/tests/test_transforms.py:116-186: (a) real weights quantised in place, (b) meta model
    + original state dict, (c) meta model + transformed state dict: identical parameters and
    buffers; outputs (a)~(b) within 1e-2 and (b)==(c)."""
    ex = ta.get_hip_nf4_executor()
    torch.manual_seed(7)
    with torch.device(dev):
        ref_m = TinyLlama().to(torch.bfloat16).eval().requires_grad_(False)
    with torch.device("meta"):
        m = TinyLlama().to(torch.bfloat16).eval().requires_grad_(False)
    for p in m.parameters():
        p._thunder_device = torch.device(dev)
    # like the reference test, the KV cache (not part of any state dict) has to be real up front
    for blk in m.layers:
        blk.k_cache, blk.v_cache = torch.zeros_like(blk.k_cache, device=dev), torch.zeros_like(blk.v_cache, device=dev)
    Q, Mat = ta.BitsAndBytesLinearQuant4bit, ta.MaterializationTransform
    jm_ref = ta.jit(ref_m, executors=(ex,), transforms=[Q()])
    jm = ta.jit(m, executors=(ex,), transforms=[Q(), Mat(dev, init=Mat.init_from_original_state_dict(ref_m.state_dict()))])
    jm2 = ta.jit(m, executors=(ex,), transforms=[Q(), Mat(dev, init=Mat.init_from_transformed_state_dict(jm_ref.state_dict()))])
    x = torch.randint(1, 255, (1, 10), device=dev)
    input_pos = torch.arange(10, device=dev)
    expected = jm_ref(x, input_pos)
    for blk in m.layers:  # jm and jm2 share m's cache buffers: start both from the same state
        blk.k_cache.zero_(), blk.v_cache.zero_()
    actual = jm(x, input_pos)
    for blk in m.layers:
        blk.k_cache.zero_(), blk.v_cache.zero_()
    actual2 = jm2(x, input_pos)
    for n, p in jm_ref.named_parameters():
        assert_close(p, jm.get_parameter(n))
        assert_close(p, jm2.get_parameter(n))
        assert jm.get_parameter(n).device.type == torch.device(dev).type
    for n, b in jm_ref.named_buffers():
        assert_close(jm.get_buffer(n), b)
        assert_close(jm2.get_buffer(n), b)
    assert jm.get_parameter("layers.0.down.weight").dtype == torch.uint8
    assert jm.get_parameter("layers.0.down.weight").shape == (64 * 1376 // 2, 1)
    assert jm.get_parameter("wte.weight").dtype == torch.bfloat16  # embeddings are not nn.Linear
    assert_close(actual, expected, rtol=1e-2, atol=1e-2)
    assert_close(actual, actual2)
    # against the unquantised module: loose, NF4 is lossy
    for blk in ref_m.layers:
        blk.k_cache.zero_(), blk.v_cache.zero_()
    assert_close(expected.float(), ref_m(x, input_pos).float(), rtol=0.3, atol=0.3)


def test_state_dict_round_trips(ta, dev):
    """thunder/tests/test_networks.py:342-357 (disabled there): transformed state dict reloads
    exactly; reloading the original state dict is idempotent; the reverse transform dequantises."""
    mlp = _mlp(dev, torch.bfloat16)
    x = torch.randn(2, 512, device=dev).to(torch.bfloat16)
    ex = ta.get_hip_nf4_executor()
    jm = ta.jit(mlp, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=(ex,))
    y = jm(x)
    sd = {k: v.clone() for k, v in jm.state_dict().items()}
    other = _mlp(dev, torch.bfloat16)
    with torch.no_grad():
        for p in other.parameters():
            p.mul_(0.5)
    jm2 = ta.jit(other, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=(ex,))
    assert not torch.equal(jm2(x), y)
    res = jm2.load_state_dict(sd)
    assert not res.missing_keys and not res.unexpected_keys
    assert torch.equal(jm2(x), y)
    with pytest.raises(RuntimeError, match="Missing key"):
        jm2.load_state_dict({k: v for k, v in sd.items() if k != "0.weight.absmax"})
    with pytest.raises(RuntimeError, match="size mismatch"):
        jm2.load_state_dict({**sd, "0.weight": sd["0.weight"][:10]})
    jm2.load_state_dict({k: v for k, v in sd.items() if k != "2.bias"}, strict=False)
    # assign=True rebinds the overrides: the next call re-plans and still gives the same numbers
    misses = ta.cache_misses(jm2)
    jm2.load_state_dict({k: v.clone() for k, v in sd.items()}, assign=True)
    assert torch.equal(jm2(x), y) and ta.cache_misses(jm2) == misses + 1
    # original (unquantised) state dict streamed through the transform
    jm2.load_original_state_dict({k: v * 0.5 for k, v in mlp.state_dict().items()})
    assert not torch.equal(jm2(x), y)
    jm2.load_original_state_dict(mlp.state_dict())
    assert torch.equal(jm2(x), y)
    for k, v in jm.state_dict().items():
        assert torch.equal(jm2.state_dict()[k], v), k
    # reverse transform: original keys, original dtype/shape, values = dequantised weights
    osd = jm.original_state_dict()
    assert list(osd) == list(mlp.state_dict())
    w = osd["0.weight"]
    assert w.dtype == torch.bfloat16 and w.shape == (1024, 512)
    assert_close(w.float(), mlp[0].weight.float(), atol=0.16 * mlp[0].weight.abs().max().item(), rtol=0)
    assert torch.equal(osd["0.bias"], mlp[0].bias)


def test_compile_spellings_and_cache(ta, dev):
    mlp = _mlp(dev, torch.bfloat16)
    x = torch.randn(1, 512, device=dev).to(torch.bfloat16)
    ex = ta.get_hip_nf4_executor()
    a = ta.jit(mlp, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=(ex,))
    b = ta.compile(mlp, plugins="quantize-int4")
    c = ta.compile(mlp, transforms=[ta.BitsAndBytesLinearQuant4bit()])
    d = ta.jit(mlp, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=["quant_hip_nf4"], check_prologue="always")
    ya = a(x)
    for j in (b, c, d):
        assert torch.equal(j(x), ya)
    assert ta.cache_misses(a) == 1 and ta.cache_hits(a) == 0
    a(x), a(x)
    assert ta.cache_misses(a) == 1 and ta.cache_hits(a) == 2 and ta.compile_stats(a).calls == 3
    # rebinding an override invalidates the plan; the prologue then checks the new tensor
    a._overrides_parameters["0.bias"] = a.get_parameter("0.bias").clone()
    a(x)
    assert ta.cache_misses(a) == 2
    a._overrides_parameters["0.weight.absmax"] = a.get_parameter("0.weight.absmax")[:5]
    with pytest.raises(AssertionError, match="shape"):
        a(x)
    with pytest.raises(TypeError):
        ta.last_traces(ta.jit(mlp))
    assert ta.compile_data(a).executors_list == (ex,)


def test_only_linear_calls_on_quantized_weights_are_rewritten(ta, dev):
    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = torch.nn.Linear(64, 32, bias=False)
            self.other = torch.nn.Parameter(torch.randn(32, 64))

        def forward(self, x):
            a = torch.nn.functional.linear(x, self.lin.weight)      # functional use of a Linear's weight
            b = torch.nn.functional.linear(x, self.other)           # not a Linear's weight: untouched
            return a, b, self.lin.weight.shape, self.lin.weight.dtype

    torch.manual_seed(0)
    with torch.device(dev):
        m = M().to(torch.bfloat16).eval().requires_grad_(False)
        x = torch.randn(3, 64).to(torch.bfloat16)
    jm = ta.jit(m, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=(ta.get_hip_nf4_executor(),))
    a, b, wshape, wdtype = jm(x)
    assert_close(a.float(), m.lin(x).float(), atol=0.5, rtol=0.5)
    assert a.shape == (3, 32) and not torch.equal(a, m.lin(x))
    assert torch.equal(b, torch.nn.functional.linear(x, m.other))
    assert tuple(wshape) == (64 * 32 // 2, 1) and wdtype == torch.uint8  # any other use sees the packed tensor


def test_double_quant_through_the_transform(ta, dev, oracle):
    """``double_quant=True`` (the reference leaves it as a TODO, thunder/transforms/quantization.py:84): absmax in 8
    bits + nested statistics as override / state-dict entries, the ``_dq`` operator in the plan, state dicts that
    round-trip, and a reverse transform that dequantises through the nested form."""
    mlp = _mlp(dev, torch.bfloat16)
    x = torch.randn(3, 512, device=dev).to(torch.bfloat16)
    ex = ta.get_hip_nf4_executor()
    tr = ta.BitsAndBytesLinearQuant4bit(double_quant=True)
    jm = ta.jit(mlp, transforms=[tr], executors=(ex,))
    plain = ta.jit(mlp, transforms=[ta.BitsAndBytesLinearQuant4bit()], executors=(ex,))
    y, y_plain = jm(x), plain(x)
    assert_close(y.float(), y_plain.float(), atol=5e-2, rtol=5e-2)   # 8-bit statistics cost a little accuracy ...
    assert not torch.equal(y, y_plain)                               # ... and are really in use
    qs = tr.quant_states["0.weight"]
    assert qs["absmax.dtype"] == torch.uint8 and qs["absmax.shape"] == (8192,) and qs["nested_blocksize"] == 256
    assert qs["nested_absmax.shape"] == (32,) and qs["nested_quant_map.shape"] == (256,) and qs["nested_offset.shape"] == (1,)
    sd = jm.state_dict()
    assert list(sd) == ["0.weight", "0.bias", "2.weight", "2.bias",
                        "0.weight.absmax", "0.weight.code", "0.weight.nested_absmax", "0.weight.nested_quant_map", "0.weight.nested_offset",
                        "2.weight.absmax", "2.weight.code", "2.weight.nested_absmax", "2.weight.nested_quant_map", "2.weight.nested_offset"]
    # the stored statistics are the oracle's compression of the plain absmax
    _, absmax = oracle.C().quantize(mlp[0].weight.cpu(), 64)
    D = oracle.create_dynamic_map()
    off = oracle.C().dq_offset(absmax)
    q, a2 = oracle.C().dq_compress(absmax, D, off)
    assert torch.equal(sd["0.weight.absmax"].cpu(), q) and torch.equal(sd["0.weight.nested_absmax"].cpu(), a2)
    assert torch.equal(sd["0.weight.nested_quant_map"].cpu(), D) and sd["0.weight.nested_offset"].cpu().tolist() == [off]
    # the plan calls the _dq operator with tensors only
    comp = ta.last_traces(jm)[-1]
    calls = [b for b in comp.bound_symbols if b.sym.name == "hip_matmul_nf4_dq"]
    assert len(calls) == 2 and not [b for b in comp.bound_symbols if b.sym.name in ("hip_matmul_nf4", "linear")]
    assert [getattr(a, "name", a) for a in calls[0].args] == [
        "t_0_input", "t_0_weight", "t_0_bias", "t_0_weight_absmax", "t_0_weight_nested_absmax", "t_0_weight_nested_quant_map",
        "t_0_weight_nested_offset", "t_0_weight_code", 64, 256, torch.bfloat16, (1024, 512)]
    assert [a.name for a in comp.args][-5:] == ["t_2_weight_absmax", "t_2_weight_code", "t_2_weight_nested_absmax",
                                                "t_2_weight_nested_quant_map", "t_2_weight_nested_offset"]
    # state dict of the transformed module reloads exactly, also into a differently initialised module
    other = _mlp(dev, torch.bfloat16)
    with torch.no_grad():
        for p in other.parameters():
            p.mul_(0.5)
    jm2 = ta.jit(other, transforms=[ta.BitsAndBytesLinearQuant4bit(double_quant=True)], executors=(ex,))
    assert not torch.equal(jm2(x), y)
    jm2.load_state_dict({k: v.clone() for k, v in sd.items()})
    assert torch.equal(jm2(x), y)                                    # includes the offset, which is cached by value
    jm2.load_original_state_dict({k: v * 0.5 for k, v in mlp.state_dict().items()})
    assert not torch.equal(jm2(x), y)
    jm2.load_original_state_dict(mlp.state_dict())
    assert torch.equal(jm2(x), y)
    # reverse transform
    osd = jm.original_state_dict()
    assert list(osd) == list(mlp.state_dict()) and osd["0.weight"].dtype == torch.bfloat16 and osd["0.weight"].shape == (1024, 512)
    assert_close(osd["0.weight"].float(), mlp[0].weight.float(), atol=0.17 * mlp[0].weight.abs().max().item(), rtol=0)


def test_lut_rounding_option(ta, dev, oracle):
    mlp = _mlp(dev, torch.bfloat16)
    jm = ta.jit(mlp, transforms=[ta.BitsAndBytesLinearQuant4bit(lut_rounding="dtype")], executors=(ta.get_hip_nf4_executor(),))
    code = jm.get_parameter("0.weight.code").cpu()
    assert torch.equal(code, oracle.nf4_lut().to(torch.bfloat16).float()) and not torch.equal(code, oracle.nf4_lut())


@pytest.mark.gpu
def test_reduce_overhead_plugin_graph_replay_equals_eager(ta):
    """``compile(model, plugins=["quantize-int4", "reduce-overhead"])``: the forward pass replays from
    a HIP graph.  Every replay (with eager work and synchronisations in between) must reproduce the
    eager result of the same jitted module for the input of that call."""
    import torch

    print("graph replay of a quantized MLP", flush=True)
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Linear(512, 1024, bias=False), torch.nn.GELU(), torch.nn.Linear(1024, 512, bias=True))
    model = model.to(dev, torch.bfloat16).requires_grad_(False)
    eager = ta.compile(model, plugins="quantize-int4")
    graphed = ta.compile(model, plugins=["quantize-int4", "reduce-overhead"])
    for i in range(6):
        g = torch.Generator(device=dev).manual_seed(100 + i)
        x = torch.randn(4, 512, generator=g, device=dev).to(torch.bfloat16)
        want = eager(x)
        got = graphed(x).clone()
        torch.cuda.synchronize()
        assert torch.equal(want, got), f"replay {i}"
        _ = (want.float() @ want.float().t()).sum().item()  # unrelated eager work between replays
    # a new input signature is a new capture
    x = torch.randn(1, 512, device=dev).to(torch.bfloat16)
    assert torch.equal(eager(x), graphed(x))


def test_thunder_adapter_is_import_guarded():
    """Where Thunder is not installed the adapter module imports fine and ``install()`` says what is
    missing; where it is installed, the returned class derives from the reference's transform."""
    import importlib

    adapter = importlib.import_module("lightning-thunder_amd.thunder_adapter")
    try:
        import thunder  # noqa: F401
    except ImportError:
        with pytest.raises(ImportError, match="lightning-thunder"):
            adapter.install()
    else:
        cls = adapter.install()
        assert cls.executor.name == adapter.EXECUTOR_NAME


def test_nested_offset_is_remembered_per_tensor_object(ta):
    """The double-quant offset is read from its one-element tensor once and kept ON that tensor: a tensor that is
    written to or rebound is read again, and a new tensor never inherits a dead one's value, even when CPython hands
    it the same id and the allocator the same address."""
    F = ta.functional
    t = torch.tensor([0.25])
    assert F._offset_value(t) == 0.25
    reads = []
    real_item = torch.Tensor.item
    try:
        torch.Tensor.item = lambda self: (reads.append(1), real_item(self))[1]
        assert F._offset_value(t) == 0.25 and not reads  # remembered: no second read
        t.fill_(0.5)  # in-place write bumps the version
        assert F._offset_value(t) == 0.5 and len(reads) == 1
        t.data = torch.tensor([0.75])  # rebound to other storage
        assert F._offset_value(t) == 0.75 and len(reads) == 2
        # a dead tensor's id and address taken by a new one with another value
        for _ in range(64):
            a = torch.tensor([1.5])
            assert F._offset_value(a) == 1.5
            ident, ptr = id(a), a.data_ptr()
            del a
            b = torch.tensor([2.5])
            same_slot = id(b) == ident and b.data_ptr() == ptr
            assert F._offset_value(b) == 2.5
            if same_slot:
                break
        assert F._offset_value(3.0) == 3.0
    finally:
        torch.Tensor.item = real_item
