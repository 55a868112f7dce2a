"""The two scenarios of the reference's own RDMA tests (python/tests/test_rdma.py:26-117 parameter server / client,
:120-200 trainer / generator), on one GPU and without actors: the same buffers, the same calls in the same order, the
same assertions on what the tensors hold afterwards.  The transport under RDMABuffer is the library's device copy."""
import pytest
import torch

from monarch_amd.staging import RDMABuffer
from util import sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class ParameterServer:  # test_rdma.py:26-47
    def __init__(self):
        g = torch.Generator().manual_seed(26)
        self.params = torch.rand(10, 10, generator=g).to(DEV)
        self.grad_buffer = torch.rand(10, 10, generator=g).to(DEV)

    def grad_handle(self) -> RDMABuffer:
        return RDMABuffer(self.grad_buffer.view(torch.uint8).flatten())

    def update(self):
        self.params += 0.01 * self.grad_buffer


class ParameterClient:  # test_rdma.py:50-66
    def __init__(self, server, buffer):
        self.server = server
        self.buffer = buffer.view(torch.uint8).flatten()

    def upload(self, tensor):
        self.server.grad_handle().write_from(tensor)

    def download(self):
        self.server.grad_handle().read_into(self.buffer)


def test_parameter_server_upload_and_download():  # test_rdma.py:95-117, the GPU half
    server = ParameterServer()
    client = ParameterClient(server, torch.ones(10, 10, device=DEV))
    assert torch.sum(client.buffer.view(torch.float32).view(10, 10)) == 100
    zeros = torch.zeros(10, 10, device=DEV)
    client.upload(zeros.view(torch.uint8).flatten())
    client.download()
    sync()
    assert torch.sum(client.buffer.view(torch.float32).view(10, 10)) == 0
    assert torch.sum(server.grad_buffer) == 0                         # the upload reached the server's own tensor
    server.grad_buffer += 3.0                                         # the server's backing buffer changes ...
    server.update()
    client.download()                                                 # ... and a download reflects it
    sync()
    assert torch.equal(client.buffer.view(torch.float32).view(10, 10), server.grad_buffer)


def test_trainer_weights_reach_the_generator_every_step():  # test_rdma.py:120-183
    trainer = torch.nn.Linear(10, 10).to(DEV)
    trainer.weight.data.zero_()
    generator = torch.nn.Linear(10, 10).to(DEV)
    handle = RDMABuffer(trainer.weight.data.view(torch.uint8).flatten())    # exchange_metadata
    for step in range(1, 4):
        trainer.weight.data.add_(1.0)                                       # weights_ready
        handle.read_into(generator.weight.data.view(torch.uint8).flatten()) # update_weights
        sync()
        assert torch.sum(generator.weight.data) == step * 100, (torch.sum(generator.weight.data), step)


def test_offsets_and_bounds_of_a_registered_buffer():
    # python/monarch/_src/tensor_engine/rdma.py:130-214: offset + size must stay inside the registered range
    backing = torch.arange(256, dtype=torch.uint8, device=DEV)
    buf = RDMABuffer(backing)
    part = torch.zeros(16, dtype=torch.uint8, device=DEV)
    assert buf.read_into(part, offset=100) == 16
    sync()
    assert part.tolist() == list(range(100, 116))
    buf.write_from(torch.full((8,), 7, dtype=torch.uint8, device=DEV), offset=248)
    sync()
    assert backing[248:].tolist() == [7] * 8 and backing[247].item() == 247
    with pytest.raises(ValueError, match="must be <="):
        buf.read_into(part, offset=241)
    with pytest.raises(ValueError, match="must be <="):
        buf.write_from(part, offset=241)


@pytest.mark.parametrize("size", [8, (1 << 20) + 5])
def test_parameter_server_example_sums_the_workers_gradient_chunks(size):
    # monarch_rdma/examples/parameter_server/parameter_server.rs: BUFFER_SIZE = 8 bytes per buffer (:89), every worker
    # computes gradient += weights + 1 (:337-343) and pushes it into its own chunk on the server (:368-370), the server adds
    # every chunk to its weights with wrapping_add and wipes the chunks (:200-206), the workers pull the weights (:411-413).
    # With N workers all bytes follow w <- w + N (w + 1) mod 256.  The server's sum is one mhip_reduce over
    # [weights, chunk_0 .. chunk_N-1], in place on the weights.
    from monarch_amd import reduce as R
    n_workers, steps = 4, 5
    ps_weights = torch.zeros(size, dtype=torch.uint8, device=DEV)
    ps_chunks = [torch.zeros(size, dtype=torch.uint8, device=DEV) for _ in range(n_workers)]
    weights_handle = RDMABuffer(ps_weights)
    grad_handles = [RDMABuffer(c) for c in ps_chunks]
    workers = [dict(weights=torch.zeros(size, dtype=torch.uint8, device=DEV), grads=torch.zeros(size, dtype=torch.uint8, device=DEV))
               for _ in range(n_workers)]
    w = 0
    for _ in range(steps):
        for rank, wk in enumerate(workers):                      # WorkerStep
            wk["grads"] += wk["weights"] + 1
            grad_handles[rank].write_from(wk["grads"])
            wk["grads"].zero_()
        R.all_reduce(ps_weights, [ps_weights] + ps_chunks, R.ReduceOp.Sum)   # PsUpdate
        for c in ps_chunks:
            c.zero_()
        for wk in workers:                                       # WorkerUpdate
            weights_handle.read_into(wk["weights"])
        sync()
        w = (w + n_workers * (w + 1)) % 256
        assert ps_weights.unique().tolist() == [w]
        for wk in workers:
            assert torch.equal(wk["weights"], ps_weights)
    assert w == (((((0 + 4) + 20) + 100) + 500) + 4 * 113) % 256    # 4, 24, 124, 112 (wrapped), 52 (wrapped)
