"""VisionTrainer: the actor body that drives the vision tower, without the Ray / DeepSpeed plumbing.

Method names, arguments, result dictionaries and error behaviour follow the reference's
python/ray/vision.py (BaseVisionTrainer / QwenVisionTrainer) and python/ray/trainer.py (Trainer):

  forward_step(iteration)        vision.py:433-500     backward_step(grad_ref)   vision.py:502-580
  optimizer_step(global_norm)    trainer.py:158-189    zero_grad()               trainer.py:278-291
  _clip_gradients                trainer.py:123-156    _build_optimizer          trainer.py:479-577
  compute_grad_norm_contribution trainer.py:334-434    get_memory_stats          trainer.py:937-953
  save/load_checkpoint           vision.py:582-657     load_pretrained_weights   vision.py:303-371

Not built (multi-process): Ray actors and object refs, CUDA-IPC hand-off, tensor / sequence parallel groups,
DeepSpeed engines.  Data comes from any iterable of batches (``set_data_iterator``) or from the synthetic
generator described by ``config["synthetic_grids"]``; the reference's HF-processor dataloader needs network
access and is outside this build.
"""

from __future__ import annotations

import logging
import math
import os
import random
import time
from collections import deque
from contextlib import nullcontext
from typing import Iterable, Iterator, Optional

import numpy as np
import torch

from .config import Qwen2_5_VLVisionConfig
from .modeling import Qwen2_5_VisionTransformerPretrainedModel
from .optim import FusedAdam, grad_norm_squared

logger = logging.getLogger(__name__)

# out_hidden_size of the published Qwen2.5-VL checkpoints (the tower is otherwise identical)
_KNOWN_OUT_HIDDEN = {"3b": 2048, "7b": 3584, "32b": 5120, "72b": 8192}


def set_seed(seed: int) -> None:
    random.seed(seed)
    np.random.seed(seed % (2**32))
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


def _lr_lambda(kind: str, warmup: int, total: int):
    """Multipliers of the usual warm-up schedules (linear / cosine / constant / constant_with_warmup)."""

    def fn(step: int) -> float:
        if kind != "constant" and step < warmup:
            return step / max(1, warmup)
        if kind in ("constant", "constant_with_warmup"):
            return 1.0
        prog = (step - warmup) / max(1, total - warmup)
        if kind == "linear":
            return max(0.0, 1.0 - prog)
        if kind == "cosine":
            return max(0.0, 0.5 * (1.0 + math.cos(math.pi * prog)))  # not clamped past the last step: the library's half cosine rises again
        raise ValueError(f"unsupported lr_scheduler_type {kind!r}")

    return fn


class Trainer:
    optimizer = None
    scheduler = None
    use_deepspeed = False
    deepspeed_engine = None

    def __init__(self, config: dict, rank: int):
        self.rank = rank
        self.config = config
        set_seed(config["seed"])

    def initialize_trainer(self) -> None:
        logger.debug("Initializing trainer %s", self.__class__.__name__)

    # ---- optimisation ------------------------------------------------------------------------------
    def _trainable_modules(self):
        for name in ("model", "projector", "lm_head"):
            mod = getattr(self, name, None)
            if mod is not None:
                yield name, mod

    def _clip_gradients(self, global_norm: float, max_norm: float) -> float:
        clip_coeff = min(1.0, max_norm / (global_norm + 1e-6))
        if clip_coeff < 1.0:
            for _, mod in self._trainable_modules():
                for p in mod.parameters():
                    if p.grad is not None:
                        p.grad.mul_(clip_coeff)
        return clip_coeff

    def _optimizer_covers_trainables(self) -> bool:
        owned = {id(p) for group in self.optimizer.param_groups for p in group["params"]}
        return all(id(p) in owned for _, mod in self._trainable_modules() for p in mod.parameters() if p.grad is not None)

    def optimizer_step(self, global_grad_norm: Optional[float] = None) -> float:
        clip_coeff = 1.0
        in_step_scale = 1.0
        if global_grad_norm is not None:
            max_norm = self.config.get("max_grad_norm", 1.0)
            if isinstance(self.optimizer, FusedAdam) and self._optimizer_covers_trainables():
                # the multi-tensor step scales the gradients itself (and stores them back scaled): one pass instead of two
                clip_coeff = in_step_scale = min(1.0, max_norm / (global_grad_norm + 1e-6))
            else:
                clip_coeff = self._clip_gradients(global_grad_norm, max_norm)
        if isinstance(self.optimizer, FusedAdam):
            self.optimizer.step(grad_scale=in_step_scale)
        elif self.optimizer is not None:
            self.optimizer.step()
        if self.scheduler is not None:
            self.scheduler.step()
        return clip_coeff

    def zero_grad(self) -> None:
        if self.optimizer is not None:
            self.optimizer.zero_grad(set_to_none=True)
            return
        for _, mod in self._trainable_modules():
            for p in mod.parameters():
                p.grad = None

    def _compute_grad_norm_squared(self, params) -> float:
        params = [p for p in params if p.grad is not None]
        if params and all(p.grad.is_cuda for p in params):
            return grad_norm_squared(params)  # two launches and one read-back for all tensors
        total = 0.0
        for p in params:  # host tensors (no GPU work to save)
            total += p.grad.detach().float().norm(2).item() ** 2
        return total

    def compute_grad_norm_contribution(self) -> dict:
        params = [p for _, mod in self._trainable_modules() for p in mod.parameters()]
        kind = self.config.get("parallelism", "none")
        norm_sq = self._compute_grad_norm_squared(params)
        if kind == "sequence":
            return {"type": "sequence", "norm_sq": norm_sq}
        if kind in ("deepspeed", "autotp"):
            return {"type": "deepspeed", "norm_sq": norm_sq}
        if kind == "tensor":  # nothing is sharded on one GPU
            return {"type": "tensor", "replicated_norm_sq": norm_sq, "sharded_norm_sq": 0.0}
        return {"type": "none", "norm_sq": norm_sq}

    def _get_decay_parameter_names(self, named_params) -> set:
        return {n for n, p in named_params if p.requires_grad and not any(x in n.lower() for x in ("bias", "norm", "ln_"))}

    def _build_optimizer(self, params, learning_rate: Optional[float] = None) -> None:
        plist = list({id(p): p for p in params}.values())
        if not plist:
            self.optimizer = None
            return
        lr = self.config["learning_rate"] if learning_rate is None else learning_rate
        wd = self.config["weight_decay"]
        # parameters on the GPU (always, once build_model has run) get the multi-tensor step; the class is a
        # torch.optim.Adam with the same groups and state, so schedulers and checkpoints do not see a difference
        Adam = FusedAdam if all(p.is_cuda for p in plist) else torch.optim.Adam
        if wd == 0.0:
            self.optimizer = Adam(plist, lr=lr, foreach=False)
            return
        named, seen = [], set()
        for mname, mod in self._trainable_modules():
            for n, p in mod.named_parameters():
                if id(p) not in seen:
                    named.append((f"{mname}.{n}", p))
                    seen.add(id(p))
        if not named:
            self.optimizer = Adam(plist, lr=lr, foreach=False)
            return
        decay_names = self._get_decay_parameter_names(named)
        decay = [p for n, p in named if p.requires_grad and n in decay_names]
        no_decay = [p for n, p in named if p.requires_grad and n not in decay_names]
        self.optimizer = Adam(
            [{"params": decay, "weight_decay": wd}, {"params": no_decay, "weight_decay": 0.0}], lr=lr, foreach=False)

    def _build_scheduler(self, num_training_steps: int) -> None:
        if self.optimizer is None:
            self.scheduler = None
            return
        ratio = self.config["warmup_ratio"]
        warmup = int(num_training_steps * ratio) if ratio > 0 else self.config["warmup_steps"]
        kind = self.config["lr_scheduler_type"]
        if kind in ("linear", "cosine", "constant", "constant_with_warmup"):
            self.scheduler = torch.optim.lr_scheduler.LambdaLR(self.optimizer, _lr_lambda(kind, warmup, num_training_steps))
            return
        # every other kind is the library's own schedule (the reference calls transformers.get_scheduler for all of
        # them, python/ray/trainer.py:579-623); the four above are restated here so that they need no library
        try:
            from transformers import get_scheduler
        except ImportError as exc:
            raise ValueError(f"lr_scheduler_type {kind!r} needs transformers.get_scheduler, which is not importable here") from exc
        self.scheduler = get_scheduler(name=kind, optimizer=self.optimizer, num_warmup_steps=warmup, num_training_steps=num_training_steps)

    # ---- helpers -----------------------------------------------------------------------------------
    def _get_torch_dtype(self, dtype_str: str = "bfloat16") -> torch.dtype:
        return {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}.get(dtype_str, torch.bfloat16)

    def _get_autocast_context(self):
        dtype = self._get_torch_dtype(self.config["dtype"])
        if self.config.get("autocast", True) and dtype != torch.float32:
            return torch.autocast(device_type="cuda", dtype=dtype, enabled=True)
        return nullcontext()

    def _get_device(self) -> torch.device:
        device = torch.device("cuda:0")
        torch.cuda.set_device(device)
        return device

    def _apply_activation_checkpointing(self, model, activation_checkpointing: bool, model_name: str = "model") -> None:
        if activation_checkpointing:
            model.gradient_checkpointing_enable()

    def get_memory_stats(self) -> dict:
        mb = 1024 * 1024
        return {"allocated_mb": torch.cuda.memory_allocated() / mb, "peak_mb": torch.cuda.max_memory_allocated() / mb}

    def reset_peak_memory(self) -> None:
        torch.cuda.reset_peak_memory_stats()


def synthetic_batches(grids, seed: int, in_features: int) -> Iterator[dict]:
    """Endless stream of batches: pixels ~ N(0,1) of shape [sum t*h*w, in_features] and their grid_thw."""
    grid = torch.tensor(grids, dtype=torch.int64).view(-1, 3)
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    gen = torch.Generator(device="cpu").manual_seed(seed)
    idx = 0
    while True:
        yield {"pixel_values": torch.randn(S, in_features, generator=gen), "image_grid_thw": grid.clone(), "sample_index": idx}
        idx += 1


class BaseVisionTrainer(Trainer):
    def __init__(self, config: dict, rank: int):
        super().__init__(config, rank)
        self.receiver_gpu_ids = None
        self.use_ipc = False
        self.model = None
        self.projector = None
        self._pending_outputs: deque = deque()
        self.sp_group = None
        self.dataloader: Optional[Iterable] = None
        self.data_iterator: Optional[Iterator] = None

    # ---- model ---------------------------------------------------------------------------------------
    def _load_model_config(self, model_name: str) -> Qwen2_5_VLVisionConfig:
        vc = self.config.get("vision_config")
        if isinstance(vc, Qwen2_5_VLVisionConfig):
            return vc
        if isinstance(vc, dict):
            return Qwen2_5_VLVisionConfig(**vc)
        low = (model_name or "").lower()
        for tag, out_hidden in _KNOWN_OUT_HIDDEN.items():
            if f"-{tag}" in low:
                return Qwen2_5_VLVisionConfig.qwen2_5_vl_tower(out_hidden_size=out_hidden)
        raise ValueError(
            f"cannot derive a vision config from model_name={model_name!r} offline; pass config['vision_config'] "
            "(a dict of Qwen2_5_VLVisionConfig fields)")

    def _create_model_instance(self, model_config):
        return Qwen2_5_VisionTransformerPretrainedModel(model_config), None

    def build_model(self) -> None:
        cfg = self.config
        parallelism = cfg["parallelism"]
        if parallelism in ("tensor", "sequence", "deepspeed", "autotp") and int(cfg.get("world_size", 1)) > 1:
            raise NotImplementedError(f"parallelism={parallelism!r} across GPUs is outside this single-GPU build")
        torch_dtype = self._get_torch_dtype(cfg["dtype"])
        if torch_dtype == torch.float16:
            raise TypeError("float16 is not built; use bfloat16 or float32")
        device = self._get_device()
        model_config = self._load_model_config(cfg.get("model_name"))
        self.model, self.projector = self._create_model_instance(model_config)
        self.model.to(torch_dtype)
        ckpt_dir = cfg.get("pretrained_checkpoint_dir")
        if ckpt_dir:
            self.load_pretrained_weights(os.path.join(ckpt_dir, "vision_model.pt"))
        self._apply_activation_checkpointing(self.model, cfg["activation_checkpointing"], "vision model")
        self.model.to(device=device, dtype=torch_dtype)
        self.model.train()
        self._build_optimizer(list(self.model.parameters()))
        self._build_scheduler(cfg["num_iterations"])

    def load_pretrained_weights(self, checkpoint_path: str) -> bool:
        if not os.path.exists(checkpoint_path):
            logger.warning("[r%d] Pretrained checkpoint not found: %s", self.rank, checkpoint_path)
            return False
        try:
            ckpt = torch.load(checkpoint_path, map_location="cpu", weights_only=True)
            state = ckpt.get("model", ckpt)
            cleaned = {}
            for key, value in state.items():
                if "attn.qkv.weight" in key or "attn.qkv.bias" in key:  # fused HF layout -> q/k/v
                    kind = "weight" if key.endswith("weight") else "bias"
                    prefix = key[: -len(f".qkv.{kind}")]
                    for name, part in zip(("q_proj", "k_proj", "v_proj"), value.chunk(3, dim=0)):
                        cleaned[f"{prefix}.{name}.{kind}"] = part
                else:
                    cleaned[key] = value
            missing, unexpected = self.model.load_state_dict(cleaned, strict=False)
            if missing:
                logger.warning("[r%d] Missing keys when loading vision weights: %s", self.rank, missing[:10])
            if unexpected:
                logger.warning("[r%d] Unexpected keys when loading vision weights: %s", self.rank, unexpected[:10])
            return True
        except Exception as exc:  # mirrors the reference: report and carry on
            logger.error("[r%d] Failed to load pretrained weights from %s: %s", self.rank, checkpoint_path, exc)
            return False

    # ---- data ----------------------------------------------------------------------------------------
    def set_data_iterator(self, loader: Iterable) -> None:
        self.dataloader = loader
        self.data_iterator = iter(loader)

    def initialize_trainer(self) -> None:
        if self.data_iterator is None:
            grids = self.config.get("synthetic_grids")
            if grids is None:
                raise ValueError("no data source: call set_data_iterator(...) or give config['synthetic_grids']")
            mc = self.model.config
            feats = mc.in_channels * mc.temporal_patch_size * mc.patch_size * mc.patch_size
            self.set_data_iterator(synthetic_batches(grids, self.config["seed"], feats))
        super().initialize_trainer()

    def set_receiver_info(self, receiver_gpu_ids, use_ipc: bool) -> None:
        self.receiver_gpu_ids = receiver_gpu_ids
        self.use_ipc = use_ipc

    # ---- steps ---------------------------------------------------------------------------------------
    def _model_forward(self, batch):
        raise NotImplementedError

    def forward_step(self, iteration: int = -1) -> dict:
        profile_time = self.config.get("profile_time", False)
        if profile_time:
            t0 = time.perf_counter()
        self._current_iteration = iteration
        try:
            batch = next(self.data_iterator)
        except StopIteration:
            self.data_iterator = iter(self.dataloader)
            batch = next(self.data_iterator)
        sample_index = batch.get("sample_index", None)
        if isinstance(sample_index, torch.Tensor):
            sample_index = sample_index.item() if sample_index.numel() == 1 else sample_index.tolist()
        device = torch.device("cuda:0")
        batch = dict(batch)
        if batch.get("pixel_values") is None and batch.get("frames") is None and batch.get("raw_images") is not None:
            # decoded still images of any size (uint8 [1, H, W, 3]): the processor's smart_resize + bicubic resize run on
            # the GPU as well (bit-identical to PIL), then the frames path below
            from .pixels import resize_frames, smart_resize

            limits = {k: int(self.config[k]) for k in ("min_pixels", "max_pixels") if self.config.get(k) is not None}
            frames = []
            for f in batch["raw_images"]:
                f = f.to(device, non_blocking=True).contiguous()
                th, tw = smart_resize(int(f.shape[1]), int(f.shape[2]), **limits)
                frames.append(resize_frames(f, th, tw))
            batch["frames"] = frames
        if batch.get("pixel_values") is None and batch.get("frames") is not None:
            # resized uint8 frames ([frames, H, W, 3] per image or video) instead of the processor's float rows: a fifth
            # of the upload; rescale / normalise / patchify run on the GPU, inside the patch-embedding GEMM
            from .pixels import grid_thw_of

            batch["frames"] = [f.to(device, non_blocking=True).contiguous() for f in batch["frames"]]
            batch["image_grid_thw"] = grid_thw_of(batch["frames"])
        else:
            batch["pixel_values"] = batch["pixel_values"].to(device, non_blocking=True)
        if not batch["image_grid_thw"].is_cuda:
            batch["image_grid_thw_host"] = batch["image_grid_thw"]  # the model plans on the host: no read-back of the device copy
        batch["image_grid_thw"] = batch["image_grid_thw"].to(device, non_blocking=True)
        vision_outputs = self._model_forward(batch)
        forward_time_ms = 0.0
        if profile_time:
            torch.cuda.synchronize()
            forward_time_ms = (time.perf_counter() - t0) * 1000
        self._pending_outputs.append(vision_outputs)
        result = {"vision_embeddings": vision_outputs, "sample_index": sample_index, "iteration": iteration,
                  "forward_time_ms": forward_time_ms}
        if self.use_ipc and self.receiver_gpu_ids is not None:
            # a receiver on the same GPU opens the embeddings in place (python/ray/vision.py:487-498): handles instead of
            # the tensor, which stays alive in _pending_outputs until its backward
            from .tensor_transfer import get_physical_gpu_id, prepare_tensor_for_transfer

            request = prepare_tensor_for_transfer(vision_outputs.detach(), receiver_gpu_ids=self.receiver_gpu_ids,
                                                  sender_gpu_id=get_physical_gpu_id(), use_ipc_if_same_gpu=True)
            result["vision_embeddings"] = request.to_dict()
        return result

    def _retrieve_gradient_tensor(self, vision_grad_ref):
        """The gradient tensor out of what the text actor returned: a tensor, ``{"grad": ...}``, or a transfer request
        whose handles are opened here (python/ray/vision.py:502-526; resolving a Ray object reference is the caller's)."""
        data = vision_grad_ref
        if isinstance(data, dict) and "grad" in data:
            data = data["grad"]
        if isinstance(data, dict) and "use_ipc" in data:
            from .tensor_transfer import TensorTransferRequest, get_physical_gpu_id, receive_tensor

            return receive_tensor(TensorTransferRequest.from_dict(data), get_physical_gpu_id())
        return data

    def _apply_vision_backward(self, vision_grad) -> None:
        if vision_grad is None:
            raise ValueError(f"[r{self.rank}] No gradient provided for backward pass")
        if not self._pending_outputs:
            raise RuntimeError(f"[r{self.rank}] No pending vision outputs available for backward pass. "
                               "Ensure forward_step was called before backward.")
        out = self._pending_outputs.popleft()
        if vision_grad.dim() == 2 and out.dim() == 3:
            if out.shape[0] != 1:
                raise RuntimeError(f"[r{self.rank}] Dimension mismatch: vision_grad is 2D {vision_grad.shape} "
                                   f"but vision_outputs has batch_size={out.shape[0]} > 1")
            vision_grad = vision_grad.unsqueeze(0)
        elif vision_grad.dim() == 3 and out.dim() == 2:
            vision_grad = vision_grad.squeeze(0)
        out.backward(gradient=vision_grad.to(device=out.device, dtype=out.dtype), retain_graph=False)

    def backward_step(self, vision_grad_ref) -> dict:
        profile_time = self.config.get("profile_time", False)
        if profile_time:
            t0 = time.perf_counter()
        self._apply_vision_backward(self._retrieve_gradient_tensor(vision_grad_ref))
        backward_time_ms = 0.0
        if profile_time:
            torch.cuda.synchronize()
            backward_time_ms = (time.perf_counter() - t0) * 1000
        return {"backward_time_ms": backward_time_ms}

    # ---- checkpoints ---------------------------------------------------------------------------------
    def save_checkpoint(self, checkpoint_dir: str, epoch: int) -> str:
        epoch_dir = os.path.join(checkpoint_dir, f"epoch_{epoch}", "vision")
        os.makedirs(epoch_dir, exist_ok=True)
        path = os.path.join(epoch_dir, f"rank_{self.rank}.pt")
        data = {"model": self.model.state_dict()}
        if self.projector is not None and self.rank == 0:
            data["projector"] = self.projector.state_dict()
        torch.save(data, path)
        return path

    def load_checkpoint(self, checkpoint_dir: str, epoch: int) -> bool:
        path = os.path.join(checkpoint_dir, f"epoch_{epoch}", "vision", f"rank_{self.rank}.pt")
        if not os.path.exists(path):
            logger.warning("[r%d] Checkpoint not found: %s", self.rank, path)
            return False
        try:
            data = torch.load(path, map_location="cpu", weights_only=True)
            if "model" in data and self.model is not None:
                self.model.load_state_dict(data["model"])
            if "projector" in data and self.projector is not None and self.rank == 0:
                self.projector.load_state_dict(data["projector"])
            return True
        except Exception as exc:
            logger.error("[r%d] Failed to load checkpoint from %s: %s", self.rank, path, exc)
            return False


class QwenVisionTrainer(BaseVisionTrainer):
    def _model_forward(self, batch):
        pixel_values, grid, host = batch.get("pixel_values"), batch["image_grid_thw"], batch.get("image_grid_thw_host")
        with self._get_autocast_context():
            if pixel_values is None:  # uint8 frames: the model makes the patch rows itself
                return self.model(frames=batch["frames"], grid_thw=grid).unsqueeze(0)
            if pixel_values.dim() == 5:  # [B, C, T, H, W] collated images that share one grid
                B = pixel_values.shape[0]
                if grid.dim() == 1:
                    grid = grid.unsqueeze(0).expand(B, -1)
                    host = None if host is None else host.unsqueeze(0).expand(B, -1)
                elif grid.dim() == 2 and grid.shape[0] != B:
                    raise ValueError(f"image_grid_thw batch dimension {grid.shape[0]} doesn't match pixel_values batch dimension {B}")
                out = self.model(hidden_states=pixel_values, grid_thw=grid, grid_thw_host=host)
                return out.reshape(B, out.shape[0] // B, -1)
            if grid.dim() == 1:
                grid = grid.unsqueeze(0)
                host = None if host is None else host.unsqueeze(0)
            return self.model(hidden_states=pixel_values, grid_thw=grid, grid_thw_host=host).unsqueeze(0)


VisionTrainer = QwenVisionTrainer
