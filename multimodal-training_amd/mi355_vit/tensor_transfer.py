"""Same-GPU, zero-copy hand-off of a tensor between two processes: the vision actor's embeddings to the text actor
and the embeddings' gradient back (python/ray/tensor_transfer.py:20-98 and :101-224 of the reference, used at
python/ray/vision.py:480-526).

The sender exports the tensor's device allocation as an inter-process memory handle together with an inter-process
event recorded on its stream; the receiver opens both, makes its stream wait for the event and works on the sender's
memory directly.  On ROCm the handles are HIP IPC handles (PyTorch's ``reduce_tensor`` / ``Event.ipc_handle``); nothing
is copied and the host does not wait.  The sender must keep the tensor alive until the receiver is done with it (the
trainer keeps its outputs queued until their backward).  Tensors on different GPUs are handed over as they are, for
the caller's own transport (the reference uses Ray's there); which actors share a GPU is the orchestrator's business
(``gather_gpu_ids`` / ``detect_collocated_actors`` of the reference need Ray and are not rebuilt).
"""

from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch


def get_physical_gpu_id() -> str:
    """UUID of the current device ("cpu" without one): what tells two processes that they share a GPU whatever their
    device numbering (python/ray/utils.py:9-22)."""
    if not torch.cuda.is_available():
        return "cpu"
    return str(torch.cuda.get_device_properties(torch.cuda.current_device()).uuid)


def create_ipc_handle(tensor: torch.Tensor) -> Tuple[Any, str, Any]:
    """(memory handle, sender's GPU id, event handle) for a GPU tensor; the event marks the point on the current stream
    where the tensor's values are complete (tensor_transfer.py:20-51)."""
    from torch.multiprocessing.reductions import reduce_tensor

    if not tensor.is_cuda:
        raise ValueError("Tensor must be on CUDA device to create IPC handle")
    tensor = tensor.contiguous()
    return reduce_tensor(tensor), get_physical_gpu_id(), _completion_event_handle()


_interprocess_events: Optional[bool] = None  # None: not tried yet on this machine


def _completion_event_handle() -> Optional[Any]:
    """Handle of an inter-process event recorded on the current stream, or None after waiting on the host instead.

    Some driver stacks have no inter-process events (recording one is refused with "invalid argument").  There the
    sender waits for its stream before it exports the memory handle, so the values are complete when the receiver opens
    it, and no event travels: one host wait per hand-off instead of a wait on the receiver's stream."""
    global _interprocess_events
    if _interprocess_events is not False:
        try:
            event = torch.cuda.Event(interprocess=True)
            torch.cuda.current_stream().record_event(event)
            handle = event.ipc_handle()
            _interprocess_events = True
            return handle
        except RuntimeError:
            if _interprocess_events:  # they worked before: a real failure
                raise
            _interprocess_events = False
    torch.cuda.current_stream().synchronize()
    return None


def reconstruct_tensor_from_ipc(ipc_handle: Any, physical_gpu_id: str, sender_gpu_id: str, event_ipc_handle: Optional[Any] = None) -> torch.Tensor:
    """The sender's tensor, opened in this process without a copy; the current stream waits for the sender's event
    first (tensor_transfer.py:54-98)."""
    if physical_gpu_id != sender_gpu_id:
        raise ValueError(f"IPC handle is for GPU {sender_gpu_id}, but receiver is on GPU {physical_gpu_id}. "
                         "CUDA IPC only works for processes on the same physical GPU.")
    device_id = torch.cuda.current_device()
    if event_ipc_handle is not None:
        remote = torch.cuda.Event.from_ipc_handle(device=device_id, handle=event_ipc_handle)
        torch.cuda.current_stream().wait_event(remote)
    func, args = ipc_handle
    args = list(args)
    args[6] = device_id  # the device ordinal in this process's numbering
    return func(*args)


class TensorTransferRequest:
    """What travels between the actors: the tensor itself, or the handles that let a process on the same GPU open it."""

    def __init__(self, tensor: Optional[torch.Tensor] = None, ipc_handle: Optional[Any] = None, sender_gpu_id: Optional[str] = None,
                 shape: Optional[Tuple] = None, dtype: Optional[torch.dtype] = None, use_ipc: bool = False, event_ipc_handle: Optional[Any] = None):
        self.tensor, self.ipc_handle, self.sender_gpu_id = tensor, ipc_handle, sender_gpu_id
        self.shape, self.dtype, self.use_ipc, self.event_ipc_handle = shape, dtype, use_ipc, event_ipc_handle

    def to_dict(self) -> Dict[str, Any]:
        return {"tensor": self.tensor, "ipc_handle": self.ipc_handle, "sender_gpu_id": self.sender_gpu_id, "shape": self.shape,
                "dtype": str(self.dtype) if self.dtype else None, "use_ipc": self.use_ipc, "event_ipc_handle": self.event_ipc_handle}

    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "TensorTransferRequest":
        dtype_str = data.get("dtype")
        dtype = getattr(torch, dtype_str.split(".")[-1]) if dtype_str else None
        return cls(tensor=data.get("tensor"), ipc_handle=data.get("ipc_handle"), sender_gpu_id=data.get("sender_gpu_id"), shape=data.get("shape"),
                   dtype=dtype, use_ipc=data.get("use_ipc", False), event_ipc_handle=data.get("event_ipc_handle"))


def prepare_tensor_for_transfer(tensor: torch.Tensor, receiver_gpu_ids: List[str], sender_gpu_id: str, use_ipc_if_same_gpu: bool = True) -> TensorTransferRequest:
    """Handles when every receiver shares the sender's GPU, the tensor itself otherwise (tensor_transfer.py:166-207)."""
    same_gpu = all(g == sender_gpu_id for g in receiver_gpu_ids)
    if same_gpu and use_ipc_if_same_gpu and tensor.is_cuda:
        handle, gpu_id, event_handle = create_ipc_handle(tensor)
        return TensorTransferRequest(ipc_handle=handle, sender_gpu_id=gpu_id, shape=tensor.shape, dtype=tensor.dtype, use_ipc=True,
                                     event_ipc_handle=event_handle)
    return TensorTransferRequest(tensor=tensor, sender_gpu_id=sender_gpu_id, shape=tensor.shape, dtype=tensor.dtype, use_ipc=False)


def receive_tensor(transfer_request: TensorTransferRequest, receiver_gpu_id: str) -> torch.Tensor:
    """tensor_transfer.py:210-224."""
    if transfer_request.use_ipc:
        return reconstruct_tensor_from_ipc(transfer_request.ipc_handle, receiver_gpu_id, transfer_request.sender_gpu_id,
                                           transfer_request.event_ipc_handle)
    return transfer_request.tensor
