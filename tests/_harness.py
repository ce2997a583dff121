"""Shared helpers of the GPU parity tests: a synthetic chunk list driven through the
product (FP16Adam over the C ABI) and mirrored on the CPU oracle."""
import numpy as np
import torch

import patrickstar_amd as ps

N_FULL = 64 * 1024 * 1024


def bits(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)


def assert_bits_equal(got, want, what):
    gb, wb = bits(np.ascontiguousarray(got)), bits(np.ascontiguousarray(want))
    if not np.array_equal(gb, wb):
        bad = np.flatnonzero(gb != wb)
        raise AssertionError(
            f"{what}: {bad.size} of {gb.size} elements differ; first at {bad[:4]}: got {got.ravel()[bad[:4]]} want {want.ravel()[bad[:4]]}"
        )


def tensor_spans(client, optimizer):
    """(chunk position, element offset, numel) of every trainable parameter, in the optimizer's own order: the
    operator calls the reference makes in one step, as the oracle wants them."""
    index = client.chunk_tensor_index
    position_of = {q.fp16: i for i, q in enumerate(client.positions())}
    out = []
    for group in optimizer.param_groups:
        for p in group["params"]:
            if p.requires_grad:
                info = index.get_tensor_info(p.ps_attr.data_id())
                out.append((position_of[info.chunk_id], info.start_offset, info.numel))
    return out


class ChunkHarness:
    """n_chunks x chunk_size synthetic chunk list on cuda:0 with an FP16Adam on top."""

    def __init__(self, n_chunks, chunk_size, loss_scaler=None, used_numel_last=None, seed=0, **adam_kwargs):
        self.device = torch.device("cuda:0")
        self.n_chunks, self.chunk_size = n_chunks, chunk_size
        self.client = ps.PatrickStarClient(0, chunk_size)
        self.params = self.client.append_flat_chunks(n_chunks, used_numel_last)
        self.opt = ps.FP16Adam(self.client, self.params, loss_scaler=loss_scaler, **adam_kwargs)
        self.gen = torch.Generator(device=self.device)
        self.gen.manual_seed(seed)
        self.used = [p.ps_attr.numel for p in self.params]

    # payload tensors of position i
    def payloads(self, i):
        pos = self.client.positions()[i]
        cl = self.client.chunk_list
        return cl[pos.fp32].payload, cl[pos.exp_avg].payload, cl[pos.exp_avg_sq].payload, cl[pos.fp16].payload

    def fill_state(self, p_std=0.02, m_std=1e-4, v_std=1e-6):
        for i in range(self.n_chunks):
            p, m, v, h = self.payloads(i)
            n = self.used[i]
            p[:n].normal_(0, p_std, generator=self.gen)
            if m_std:
                m[:n].normal_(0, m_std, generator=self.gen)
            if v_std:
                v[:n].normal_(0, v_std, generator=self.gen).abs_()
            h[:n].copy_(p[:n])

    def fill_grads(self, std, scale):
        for i in range(self.n_chunks):
            h = self.payloads(i)[3]
            n = self.used[i]
            tmp = torch.empty(n, device=self.device).normal_(0, std, generator=self.gen).mul_(scale)
            h[:n].copy_(tmp)  # fp32 -> fp16 RNE
            h[n:].zero_()

    def download(self, i):
        # always a private copy: a host-resident payload would otherwise be aliased by ".cpu()"
        return tuple(t.detach().to("cpu", copy=True).numpy() for t in self.payloads(i))

    def oracle_chunks(self, indices=None):
        """Host mirror of the current device state, as the oracle's chunk dicts."""
        out = []
        for i in indices if indices is not None else range(self.n_chunks):
            p, m, v, h = self.download(i)
            out.append({"p32": p, "m": m, "v": v, "p16": h})
        return out

    def compare(self, oracle_chunks, indices=None, what=""):
        for k, i in enumerate(indices if indices is not None else range(self.n_chunks)):
            p, m, v, h = self.download(i)
            oc = oracle_chunks[k]
            assert_bits_equal(p, oc["p32"], f"{what} chunk {i} fp32 param")
            assert_bits_equal(m, oc["m"], f"{what} chunk {i} exp_avg")
            assert_bits_equal(v, oc["v"], f"{what} chunk {i} exp_avg_sq")
            assert_bits_equal(h, oc["p16"], f"{what} chunk {i} fp16 param")


class HybridHarness(ChunkHarness):
    """Like ChunkHarness, with some positions kept in pinned host memory."""

    def __init__(self, n_chunks, chunk_size, host_positions, loss_scaler=None, seed=0, host_keeps_fp16=True,
                 **adam_kwargs):
        self.device = torch.device("cuda:0")
        self.n_chunks, self.chunk_size = n_chunks, chunk_size
        host = set(host_positions)
        self.client = ps.PatrickStarClient(
            0, chunk_size, config={"host_chunk_policy": lambda pos: pos in host, "host_keeps_fp16": host_keeps_fp16}
        )
        self.params = self.client.append_flat_chunks(n_chunks)
        self.opt = ps.FP16Adam(self.client, self.params, loss_scaler=loss_scaler, **adam_kwargs)
        self.gen = torch.Generator(device=self.device)
        self.gen.manual_seed(seed)
        self.used = [p.ps_attr.numel for p in self.params]

    def fill_state(self):
        for i in range(self.n_chunks):
            p, m, v, h = self.payloads(i)
            n = self.chunk_size
            p.copy_(torch.empty(n, device=self.device).normal_(0, 0.02, generator=self.gen))
            m.copy_(torch.empty(n, device=self.device).normal_(0, 1e-4, generator=self.gen))
            v.copy_(torch.empty(n, device=self.device).normal_(0, 1e-6, generator=self.gen).abs_())
            h.copy_(p)
        torch.cuda.synchronize()

    def fill_grads(self, std, scale):
        for i in range(self.n_chunks):
            h = self.payloads(i)[3]
            tmp = torch.empty(self.chunk_size, device=self.device).normal_(0, std, generator=self.gen).mul_(scale).half()
            h.copy_(tmp)
        torch.cuda.synchronize()


def new_grads_like(gen_np, n, std, scale):
    return (gen_np.normal(0, std, n).astype(np.float32) * np.float32(scale)).astype(np.float16)
