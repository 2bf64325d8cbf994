"""Single-GPU counterpart of the reference's inference entry point, so code
written against `landmark.init_inference` drives the HIP renderer unchanged.

  init_inference            landmark/__init__.py:61-92 (config normalisation, sanity checks :47-58)
  InferenceModuleInitializer landmark/render/util/initializer.py:6-44 (model construction from the config)
  InferenceInterface/Module landmark/render/util/inference_module.py:26-170 (preprocess / forward / postprocess)
  InferenceEngine           landmark/render/inference_engine/inference_engine.py:31-138
                            (checkpoint load, runtime switch, instruction list)

What is kept: the call protocol (`engine(*args)` runs preprocess -> forward ->
postprocess under `no_grad`, a non-tuple forward result is wrapped in a tuple
before postprocess), checkpoint loading through the model's own
`get_state_dict_from_ckpt` / `load_from_state_dict`, the `runtime` and
`kernel_fusion` switches and the reference's sanity assertions.  What is not:
data / tensor parallel ranks and CPU<->GPU block offload.  A parallel
configuration that asks for more than one rank raises; the reference itself
refuses offload for Gaussian models (initializer.py:26-27).
"""
from enum import Enum
from pathlib import Path
from typing import Any, Dict, Mapping, Optional, Union  # noqa: F401

import torch
from torch import nn


class Config(dict):
    """Attribute-addressable dict (the reference's `landmark.utils.Config`); nested dicts convert on access."""

    def __getattr__(self, name):
        try:
            value = self[name]
        except KeyError:
            raise AttributeError(name) from None
        if isinstance(value, dict) and not isinstance(value, Config):
            value = self[name] = Config(value)
        return value

    def __setattr__(self, name, value):
        self[name] = value

    @classmethod
    def from_file(cls, path):
        """A Python config file: its public top-level names become the fields."""
        import runpy
        scope = runpy.run_path(str(path))
        return cls({k: v for k, v in scope.items() if not k.startswith("_")})


class RuntimeType(Enum):
    Kernel = "Kernel"
    Torch = "Torch"


def _as_config(config):
    if config is None or isinstance(config, Config):
        return config
    if isinstance(config, dict):
        return Config(config)
    if isinstance(config, (str, Path)):
        return Config.from_file(config)
    return config  # any attribute-addressable object (a dataclass, the reference's BaseConfig)


def _get(config, name, default=None):
    if config is None:
        return default
    if isinstance(config, dict):
        return config.get(name, default)
    return getattr(config, name, default)


def _set(config, name, value):
    if isinstance(config, dict):
        config[name] = value
    else:
        setattr(config, name, value)


def _has(config, name):
    return _get(config, name, None) is not None


class InferenceInterface(nn.Module):
    """preprocess / forward / postprocess protocol (inference_module.py:26-40)."""

    def preprocess(self, *args, **kwargs):
        return args, kwargs

    def postprocess(self, *args, **kwargs):
        return args, kwargs


class InferenceModule(InferenceInterface):
    """Wraps a model and forwards the protocol to it (inference_module.py:43-170).  Subclasses build their model
    in `__init__` and may override the three stages."""

    def __init__(self, model: Optional[nn.Module] = None) -> None:
        super().__init__()
        self.model = model

    @property
    def inter_model(self):
        return self.model

    @inter_model.setter
    def inter_model(self, model):
        self.model = model

    def get_state_dict_from_ckpt(self, file_path, map_location) -> Mapping[str, Any]:
        return self.model.get_state_dict_from_ckpt(file_path, map_location)

    def load_from_state_dict(self, state_dict: Mapping[str, Any], strict: bool = False):
        self.model.load_from_state_dict(state_dict, strict)

    def preprocess(self, *args, **kwargs):
        if self.model is None or not hasattr(self.model, "preprocess"):
            return super().preprocess(*args, **kwargs)
        return self.model.preprocess(*args, **kwargs)

    def postprocess(self, *args, **kwargs):
        if self.model is None or not hasattr(self.model, "postprocess"):
            return _plain_postprocess(*args, **kwargs)
        return self.model.postprocess(*args, **kwargs)

    def forward(self, *args, **kwargs):
        assert self.model is not None
        return self.model(*args, **kwargs)


def _plain_preprocess(*args, **kwargs):
    return args, kwargs


def _plain_postprocess(*args, **kwargs):
    # inference_module.py:13-16: a single positional result is returned bare
    if len(args) == 1 and not kwargs:
        return args[0]
    return args + (kwargs,) if kwargs else args


def _sanity_check(model_config, inference_config):
    # landmark/__init__.py:47-58
    if _has(model_config, "act_cache") and _has(inference_config, "offload_config"):
        assert model_config.act_cache is False, "Offload is not supportted when act_cache is True"
    if _has(inference_config, "half_precision"):
        assert inference_config.half_precision is False, "Half precision is not supportted yet"
    if _has(inference_config, "static_allocation"):
        assert inference_config.static_allocation is False, "Static Allocation is not supportted yet"


def _single_rank_only(parallel_config):
    for name in ("tp_size", "dp_size", "world_size"):
        n = _get(parallel_config, name, 1)
        if n is not None and int(n) > 1:
            raise NotImplementedError("%s=%d: this build renders on one GPU per process" % (name, int(n)))


class InferenceEngine(nn.Module):
    """Loads the checkpoint into the model, moves it to the GPU and runs the three stages per call."""

    def __init__(self, model: nn.Module, config) -> None:
        super().__init__()
        self.model = model
        if not isinstance(model, InferenceModule):
            assert not (hasattr(model, "preprocess") or hasattr(model, "postprocess"))
            object.__setattr__(model, "preprocess", _plain_preprocess)
            object.__setattr__(model, "postprocess", _plain_postprocess)
            self.base_model = model
        else:
            self.base_model = model.inter_model
        self._config = config
        if _has(config, "parallel_config"):
            _single_rank_only(config.parallel_config)
        if _has(config, "offload_config"):
            raise NotImplementedError("CPU<->GPU block offload is not part of this build")
        self.runtime = RuntimeType(_get(config, "runtime", "Kernel"))  # ValueError on an unknown runtime
        self.kernel_fusion = bool(_get(config, "kernel_fusion", self.runtime is RuntimeType.Kernel))
        self._inference_output = None
        self.model.eval()
        ckpt_path = _get(config, "ckpt_path")
        if ckpt_path is not None:
            merged = self.model.get_state_dict_from_ckpt(ckpt_path, "cpu")
            self.model.load_from_state_dict(merged)
        if not torch.cuda.is_available():
            raise RuntimeError("InferenceEngine needs a GPU: the renderer has no CPU path")
        self.model.to("cuda")
        self.model.eval()

    @torch.no_grad()
    def forward(self, *args, **kwargs):
        args, kwargs = self.model.preprocess(*args, **kwargs)
        outputs = self.model.forward(*args, **kwargs)
        if not isinstance(outputs, tuple):
            outputs = (outputs,)
        self._inference_output = self.model.postprocess(*outputs)
        return self._inference_output


def render_trajectory(model, cameras, in_flight: int = 2, **forward_kwargs):
    """Render `cameras` in order with up to `in_flight` frames on the GPU at once, yielding the images in order.

    Frames are independent, and their stages stress different parts of the chip (the per-Gaussian stage is bound
    by memory bandwidth, blending by the vector units), so letting the next frame start while the current one is
    still blending raises throughput (about 7 % at 6 M Gaussians, 1080p) at the price of one frame of latency.
    Each frame runs on its own stream (and therefore its own rasterizer workspace); a yielded image is ordered
    into the caller's current stream, so it can be used like the result of a plain `model(camera)` call."""
    from collections import deque

    if in_flight < 1:
        raise ValueError("in_flight must be >= 1")
    device = next(model.parameters()).device
    caller = torch.cuda.current_stream(device)
    streams = [torch.cuda.Stream(device=device) for _ in range(in_flight)]
    pending = deque()

    def hand_over(item):
        image, done = item
        caller.wait_event(done)
        image.record_stream(caller)
        return image

    try:
        with torch.no_grad():
            for k, camera in enumerate(cameras):
                stream = streams[k % in_flight]
                stream.wait_stream(caller)  # whatever produced the model's inputs has been enqueued before
                with torch.cuda.stream(stream):
                    image = model(camera, **forward_kwargs)
                    done = torch.cuda.Event()
                    done.record(stream)
                pending.append((image, done))
                if len(pending) >= in_flight:
                    yield hand_over(pending.popleft())
            while pending:
                yield hand_over(pending.popleft())
    finally:
        from . import pipeline
        for stream in streams:  # the streams retire with this call: so do their rasterizer workspaces
            pipeline.release_workspace(device, stream)


def init_inference(based_model_cls, infer_model_cls, model_config: Union[str, Path, Config, Dict, None],
                   inference_config: Union[str, Path, Config, Dict]) -> InferenceEngine:
    """Build the model from `model_config`, wrap it in the engine described by `inference_config`.

    `model_config.ckpt` names the checkpoint (`point_cloud.ply`, with `state_dict.th` beside it);
    `inference_config` holds `runtime` ("Kernel" | "Torch"), optionally `kernel_fusion`, `ckpt_path`,
    `parallel_config` (one rank only)."""
    inference_config = _as_config(inference_config)
    model_config = _as_config(model_config)
    if _has(inference_config, "parallel_config"):
        _single_rank_only(inference_config.parallel_config)
    _sanity_check(model_config, inference_config)
    if model_config is not None:
        assert _get(model_config, "ckpt") is not None, "should set the checkpoint file path"
        if _has(inference_config, "ckpt_path"):
            assert _get(inference_config, "ckpt_path") == _get(model_config, "ckpt")
        else:
            _set(inference_config, "ckpt_path", _get(model_config, "ckpt"))
        kwargs = {"config": model_config, "scene_manager": None}
    else:
        kwargs = based_model_cls.get_kwargs() if hasattr(based_model_cls, "get_kwargs") else {}
        if not _has(inference_config, "ckpt_path"):
            _set(inference_config, "ckpt_path", None)
    model = infer_model_cls(**kwargs) if infer_model_cls is not None else based_model_cls(**kwargs)
    return InferenceEngine(model, inference_config)
