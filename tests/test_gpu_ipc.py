"""Two processes on one GPU: the vision actor hands its embeddings to a second process (a stand-in for the text actor)
through inter-process memory and event handles, the second process hands the embeddings' gradient back the same way
(python/ray/tensor_transfer.py:20-98, python/ray/vision.py:480-526).  The result must be bit-equal to the same step with
both ends in one process."""

import gc
import os
import subprocess
import sys
import tempfile
from multiprocessing.connection import Listener
from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = Path(__file__).resolve().parent.parent

# the text actor's side: open the embeddings in place, derive a gradient from them on this process's own stream, export it
PEER = r"""
import sys
from multiprocessing.connection import Client
sys.path.insert(0, sys.argv[2]); sys.path.insert(0, sys.argv[3])
import torch
from mi355_vit.tensor_transfer import TensorTransferRequest, get_physical_gpu_id, prepare_tensor_for_transfer, receive_tensor
torch.cuda.set_device(0)
conn = Client(sys.argv[1], family="AF_UNIX", authkey=b"mvit")
keep = []
while True:
    if not conn.poll(120):
        break
    msg = conn.recv()
    if msg is None:
        break
    request = TensorTransferRequest.from_dict(msg)
    emb = receive_tensor(request, get_physical_gpu_id())
    assert emb.is_cuda and tuple(emb.shape) == tuple(request.shape) and emb.dtype == request.dtype
    grad = (emb.float() * 0.5 + 1.0).to(emb.dtype)
    keep.append(grad)  # the sender of a tensor keeps it alive until the receiver is done
    back = prepare_tensor_for_transfer(grad, [request.sender_gpu_id], get_physical_gpu_id())
    checksum = float(emb.double().sum())
    del emb  # released before the answer leaves, so the sender finds nothing of its own still open here
    conn.send({"grad": back.to_dict(), "checksum": checksum, "peer_gpu": get_physical_gpu_id()})
conn.close()
"""


def _config():
    return dict(seed=5, model_name="unit-test", parallelism="none", dtype="bfloat16", attention_backend="flash_attention_2",
                activation_checkpointing=False, autocast=True, learning_rate=1e-2, weight_decay=0.01, warmup_ratio=0.0, warmup_steps=0,
                lr_scheduler_type="cosine", num_iterations=10, max_grad_norm=1.0, profile_time=False,
                vision_config=dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=128, fullatt_block_indexes=[1]),
                synthetic_grids=[[1, 16, 16], [1, 8, 24]])


def _trainer():
    from mi355_vit.trainer import VisionTrainer

    tr = VisionTrainer(_config(), rank=0)
    tr.build_model()
    tr.initialize_trainer()
    tr.zero_grad()
    return tr


def test_embeddings_and_gradient_cross_a_process_boundary_without_a_copy():
    print("[case] same-GPU hand-off between two processes: embeddings out, gradient back", flush=True)
    from mi355_vit.tensor_transfer import get_physical_gpu_id

    # both ends in this process: two steps on consecutive batches
    tr = _trainer()
    ref_checksums, ref_grads = [], []
    for step in range(2):
        tr.zero_grad()
        emb = tr.forward_step(iteration=step)["vision_embeddings"]
        assert isinstance(emb, torch.Tensor)
        ref_checksums.append(float(emb.detach().double().sum()))
        tr.backward_step({"grad": (emb.detach().float() * 0.5 + 1.0).to(emb.dtype)})
        torch.cuda.synchronize()
        ref_grads.append({n: p.grad.detach().clone() for n, p in tr.model.named_parameters()})
    del tr, emb

    sock = os.path.join(tempfile.mkdtemp(prefix="mvit_ipc_"), "s")
    env = dict(os.environ, HSA_ENABLE_IPC_MODE_LEGACY=os.environ.get("HSA_ENABLE_IPC_MODE_LEGACY", "0"))
    with Listener(sock, family="AF_UNIX", authkey=b"mvit") as listener:
        peer = subprocess.Popen([sys.executable, "-c", PEER, sock, str(ROOT), str(ROOT / "multimodal-training_amd")], env=env)
        try:
            listener._listener._socket.settimeout(180)  # the peer's first import of torch can take a minute on a fresh box
            conn = listener.accept()
            tr = _trainer()
            tr.set_receiver_info([get_physical_gpu_id()], use_ipc=True)
            for step in range(2):  # twice: a second hand-off while the first one's allocations are still open in the peer
                tr.zero_grad()
                res = tr.forward_step(iteration=step)
                handles = res["vision_embeddings"]
                assert isinstance(handles, dict) and handles["use_ipc"] and handles["tensor"] is None
                print(f"[ipc] step {step}: completion travels as {'an inter-process event' if handles['event_ipc_handle'] is not None else 'a host wait on the sender (no inter-process events on this stack)'}", flush=True)
                conn.send(handles)
                assert conn.poll(120), "the peer did not answer"
                answer = conn.recv()
                assert answer["peer_gpu"] == get_physical_gpu_id()
                here = float(tr._pending_outputs[-1].detach().double().sum())
                print(f"[ipc] step {step}: checksum of the embeddings: peer {answer['checksum']!r}, this process {here!r}, one-process run {ref_checksums[step]!r}", flush=True)
                assert answer["checksum"] == here  # the peer read the very values this process computed
                assert here == ref_checksums[step]
                assert answer["grad"]["use_ipc"]
                tr.backward_step(answer)  # {"grad": transfer request}
                torch.cuda.synchronize()
                for n, p in tr.model.named_parameters():
                    assert torch.equal(p.grad, ref_grads[step][n]), (step, n)
            # nothing of the peer's stays open here when the peer ends: a producer that exits first complains
            del answer, res, handles
            tr = None
            gc.collect()
            torch.cuda.ipc_collect()
            conn.send(None)
            conn.close()
            assert peer.wait(timeout=60) == 0
        finally:
            if peer.poll() is None:
                peer.kill()


def test_a_receiver_on_another_gpu_is_refused_and_other_gpus_get_the_tensor_itself():
    from mi355_vit.tensor_transfer import (create_ipc_handle, get_physical_gpu_id, prepare_tensor_for_transfer, receive_tensor,
                                           reconstruct_tensor_from_ipc)

    t = torch.arange(12, device=DEV, dtype=torch.float32)
    here = get_physical_gpu_id()
    plain = prepare_tensor_for_transfer(t, ["some-other-gpu"], here)
    assert not plain.use_ipc and plain.tensor is t and receive_tensor(plain, "some-other-gpu") is t
    # (nobody opens this handle, so PyTorch's sender-side accounting reports an unreleased shared tensor when the test
    # process ends; that line on stderr is about this request and nothing else)
    shared = prepare_tensor_for_transfer(t, [here], here)
    assert shared.use_ipc and shared.tensor is None and shared.shape == t.shape
    with pytest.raises(ValueError, match="only works for processes on the same physical GPU"):
        reconstruct_tensor_from_ipc(shared.ipc_handle, "some-other-gpu", here, shared.event_ipc_handle)
    with pytest.raises(ValueError, match="must be on CUDA device"):
        create_ipc_handle(torch.zeros(3))
