"""``initialize_engine(model_func, local_rank, config)`` -> ``(engine, optimizer)`` for one MI355X.

Only the configuration surface and the optimizer / loss-scaler wiring of
``patrickstar/runtime/__init__.py:40-93`` and ``patrickstar/runtime/engine.py:45-132,204-224``
are kept; the reference's hook-driven chunk movement, memory tracer and
collectives are not part of this path.  With 288 GB of HBM every chunk stays
resident: module parameters are fp16 views into the fp16 chunk payloads, so
forward and backward are ordinary PyTorch; during ``backward`` each gradient is
written over its parameter's chunk slot as soon as it is complete, probed for
inf/nan in the same pass (one fused kernel per parameter, no host sync), which
is the state ``optimizer.step()`` expects.
"""
import torch

from . import _lib
from .chunk_layout import is_param_registered
from .client import PatrickStarClient
from .fp16_adam import FP16Adam
from .loss_scaler import DynamicLossScaler, LossScaler

DEFAULT_CHUNK_SIZE = 32 * 1024 * 1024


def default_optim_config():
    return {
        "type": "Adam",
        "params": {"lr": 0.01, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0, "use_hybrid_adam": True},
    }


def parse_config(config):
    """Config dict -> (optimizer type, optimizer params, loss scaler, gradient clipping).

    Same defaults, checks and quirks as the reference engine: the fp16 block's
    ``hysteresis`` value is handed to the scaler as its ``scale_factor``,
    ``delayed_shift`` is left at 1, ``loss_scale_window`` defaults to 2000.
    """
    default = default_optim_config()
    if config is None:
        return default["type"], default["params"], None, -1
    optim_config = config.get("optimizer", default)
    optim_type = optim_config.get("type", default["type"])
    if optim_type not in ["Adam", "AdamW"]:
        raise ValueError(f"Only support Adam and AdamW at the moment. Get optimizer type {optim_type}")
    optim_params = optim_config.get("params", default["params"])
    for key, val in default["params"].items():
        if key not in optim_params:
            optim_params[key] = val

    if "fp16" not in config:
        loss_scaler = None
    else:
        fp16 = config["fp16"]
        assert fp16["enabled"], "Must enable fp16 training."
        assert "loss_scale" in fp16, "Must have `loss_scale` field set."
        if fp16["loss_scale"] == 0:
            loss_scaler = DynamicLossScaler(
                init_scale=2 ** fp16.get("initial_scale_power", 16),
                scale_factor=fp16.get("hysteresis", 2),
                scale_window=fp16.get("loss_scale_window", 2000),
                min_scale=fp16.get("min_loss_scale", 1),
            )
        else:
            loss_scaler = LossScaler(fp16["loss_scale"])
    gradient_clipping = config["gradient_clipping"] if "gradient_clipping" in config else -1
    return optim_type, optim_params, loss_scaler, gradient_clipping


class PatrickStarEngine(torch.nn.Module):
    def __init__(self, model, client, config):
        super().__init__()
        self.module = model
        self.module.train()
        self.client = client
        optim_type, optim_params, self.loss_scaler, self.gradient_clipping = parse_config(config)
        # parameters already live in the fp16 chunks on the device; buffers follow them (runtime/engine.py:134-138)
        for buffer in model.buffers():
            buffer.data = buffer.data.to(self.client.device)
        self.optimizer = FP16Adam(
            self.client,
            self.module.parameters(),
            loss_scaler=self.loss_scaler,
            gradient_clipping=self.gradient_clipping,
            lr=optim_params["lr"],
            betas=optim_params["betas"],
            eps=optim_params["eps"],
            weight_decay=optim_params["weight_decay"],
            use_adamw=(optim_type == "AdamW"),
            use_hybrid_adam=optim_params["use_hybrid_adam"],
            scan_in_step=False,  # backward() probes while it copies the gradients
            # optional key, absent from the reference's schema: "operator" (default) or "torch"
            arithmetic=optim_params.get("arithmetic", "operator"),
        )
        self.client.init(self.module, self.optimizer)
        self.iteration_cnt_ = 0
        self._copied = set()  # parameters whose gradient already sits in its chunk slot (this backward)
        for p in self.client.chunk_based_param_fp16:
            if p.requires_grad:
                p.register_post_accumulate_grad_hook(self._on_gradient_ready)

    def forward(self, *inputs, **kwargs):
        return self.module(*inputs, **kwargs)

    # -- backward-side producer ---------------------------------------------------------
    def _gradient_to_chunk(self, p):
        """Write ``p.grad`` over ``p``'s fp16 chunk slot, probing it for inf/nan in the same pass, and drop it."""
        g = p.grad if p.grad.is_contiguous() else p.grad.contiguous()
        if g.dtype not in (torch.half, torch.float):
            raise TypeError(f"gradient dtype {g.dtype} is not supported")
        scaler = self.loss_scaler
        state_ptr = scaler.state_ptr if isinstance(scaler, DynamicLossScaler) else None
        slot = self.client.access_data(p)
        with torch.cuda.device(self.client.device):
            _lib.check(
                _lib.load().ps_grad_to_chunk(
                    g.data_ptr(), int(g.dtype == torch.half), slot.data_ptr(), g.numel(), state_ptr,
                    _lib.current_stream_handle(),
                ),
                "ps_grad_to_chunk",
            )
        p.grad = None

    def _on_gradient_ready(self, p):
        """Post-accumulate-grad hook: runs during backward, as soon as ``p``'s gradient is complete (every use of the
        parameter has been differentiated, so nothing in the rest of backward reads its value any more).  The
        reference does the same copy in its post-backward module hook (``patrickstar/core/hook.py:200-230``); the
        copies overlap the rest of backward and no second full set of gradients stays alive."""
        self._gradient_to_chunk(p)
        self._copied.add(p)

    def _finish_gradients(self):
        """After backward: parameters whose hook did not fire (no gradient this iteration, or a gradient that was
        assigned by hand)."""
        for p in self.client.chunk_based_param_fp16:
            if p in self._copied:
                continue
            if not p.requires_grad:
                # a frozen parameter: the optimizer skips it (fp16_cpu_adam.py:566-569), its slot keeps the parameter
                continue
            if p.grad is not None:
                self._gradient_to_chunk(p)
            else:
                # the slot still holds the fp16 parameter, which step() would read as a gradient
                self.client.access_data(p).zero_()
        self._copied.clear()

    def backward(self, loss):
        self.optimizer.zero_grad()
        self._copied.clear()
        if self.loss_scaler:
            self.loss_scaler.backward(loss)
        else:
            loss.backward()
        self._finish_gradients()
        self.iteration_cnt_ += 1


    # -- model checkpoint -------------------------------------------------------------------
    def state_dict(self, destination=None, prefix="", keep_vars=False):
        """The model's checkpoint under the module's own parameter names, as the reference writes it
        (``patrickstar/runtime/checkpoint.py:39-88``): for every chunk-based parameter the fp32 MASTER copy (which
        is what training continues from), not the fp16 working copy; buffers as they are.  Values are CPU clones."""
        out = self.module.state_dict(prefix=prefix, keep_vars=False) if destination is None else destination
        if destination is not None:
            self.module.state_dict(destination=out, prefix=prefix, keep_vars=False)
        for key in list(out.keys()):
            out[key] = out[key].detach().to("cpu", copy=True)
        for name, p in self.module.named_parameters():
            if is_param_registered(p) and p in self.client.param_fp16_to_param_fp32_map:
                master = self.client.access_data(self.client.param_fp16_to_param_fp32_map[p])
                out[prefix + name] = master.detach().to("cpu", copy=True)
        return out

    def load_state_dict(self, state_dict, strict=False):
        """Load a checkpoint written by ``state_dict``: fp32 masters are restored and the fp16 working copies are
        refreshed from them (round to nearest even); buffers go through ``nn.Module``.  ``strict`` raises on missing
        or unexpected keys, as ``patrickstar/runtime/checkpoint.py:198-262`` does."""
        named = dict(self.module.named_parameters())
        rest = {}
        missing = [k for k in named if k not in state_dict]
        with torch.no_grad():
            for key, value in state_dict.items():
                p = named.get(key)
                if p is not None and is_param_registered(p) and p in self.client.param_fp16_to_param_fp32_map:
                    master = self.client.access_data(self.client.param_fp16_to_param_fp32_map[p])
                    master.copy_(value.to(master.device, torch.float).view(master.shape))
                    self.client.access_data(p).copy_(master)
                else:
                    rest[key] = value
        result = self.module.load_state_dict(rest, strict=False)
        unexpected = list(result.unexpected_keys)
        missing += [k for k in result.missing_keys if k not in named]
        if strict and (unexpected or missing):
            raise RuntimeError(f"Failed to load model strictly. missing: {missing} unexpected: {unexpected}")
        return result


def initialize_engine(model_func, local_rank, config=None, client=None):
    """Build the model inside a chunk client and wrap it.

    Returns ``(engine, optimizer)``.  ``model_func`` is a callable returning an
    ``nn.Module`` (or an ``nn.Module`` whose parameters were already registered
    with ``client``).
    """
    if isinstance(model_func, torch.nn.Module):
        assert client is not None, "Must pass the client when passing a nn.Module."
        model = model_func
    else:
        assert callable(model_func), "model_func need to be callable."
        cfg = config if config is not None else {}
        default_chunk_size = cfg.get("default_chunk_size", DEFAULT_CHUNK_SIZE)
        client = PatrickStarClient(rank=local_rank, default_chunk_size=default_chunk_size, config=cfg.get("client", None))
        # hybrid Adam (optimizer state of some chunk positions in host memory) is the optimizer's switch; the client
        # needs it when it places the payloads
        client.use_hybrid_adam = bool(parse_config(config)[1].get("use_hybrid_adam", True))
        model = model_func()
        # "use_cpu_embedding" (the reference's default is True, patrickstar/runtime/__init__.py:62-69; here it has to
        # be asked for): embedding weights stay fp32 parameters of PyTorch's own and are updated from fp32 gradients
        client.register_model(model, use_cpu_embedding=bool(cfg.get("use_cpu_embedding", False)))
    engine = PatrickStarEngine(model=model, client=client, config=config)
    client.start_mem_tracer()
    return (engine, engine.optimizer)
