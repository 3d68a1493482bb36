"""Calls libi6fbw.so through the C ABI on torch-owned device buffers."""
import numpy as np
import torch

from i6_native_ops_amd import cabi


class DeviceProblem:
    def __init__(self, am, edges, weights, start_end, seq_lens, n_states, device="cuda:0"):
        self.T, self.B, self.F = am.shape
        self.E = int(edges.shape[1])
        self.n_states = int(n_states)
        dev = torch.device(device)
        self.am = torch.from_numpy(np.ascontiguousarray(am)).to(dev)
        self.edges = torch.from_numpy(np.ascontiguousarray(edges)).to(dev)
        self.weights = torch.from_numpy(np.ascontiguousarray(weights)).to(dev)
        self.start_end = torch.from_numpy(np.ascontiguousarray(start_end)).to(dev)
        self.seq_lens = torch.from_numpy(np.ascontiguousarray(seq_lens)).to(dev)
        self.out = torch.empty((self.T, self.B, self.F), dtype=torch.float32, device=dev)
        self.loss = torch.empty((self.T, self.B), dtype=torch.float32, device=dev)
        self.ws_bytes = cabi.workspace_size(self.T, self.B, self.F, self.E, self.n_states)
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev)

    def run(self, out_mode=cabi.OUT_NEG_LOG, check=True, input_flags=None):
        stream = torch.cuda.current_stream().cuda_stream
        if input_flags is None:
            cabi.run(self.am.data_ptr(), self.am.stride(0), self.am.stride(1), self.edges.data_ptr(),
                     self.edges.stride(0) if self.E > 0 else 0, self.weights.data_ptr(), self.start_end.data_ptr(),
                     self.start_end.stride(0), self.seq_lens.data_ptr(), self.T, self.B, self.F, self.E, self.n_states,
                     out_mode, self.out.data_ptr(), self.loss.data_ptr(), self.ws.data_ptr(), self.ws_bytes, stream)
        else:
            cabi.run_strided(self.am.data_ptr(), self.am.stride(0), self.am.stride(1), input_flags, self.edges.data_ptr(),
                             self.edges.stride(0) if self.E > 0 else 0, self.weights.data_ptr(), self.start_end.data_ptr(),
                             self.start_end.stride(0), self.seq_lens.data_ptr(), self.T, self.B, self.F, self.E,
                             self.n_states, out_mode, self.out.data_ptr(), self.out.stride(0), self.out.stride(1),
                             self.loss.data_ptr(), self.ws.data_ptr(), self.ws_bytes, stream)
        if check:
            code, seq = cabi.read_status(self.ws.data_ptr(), self.B, stream)
            if code != 0:
                raise cabi.FbwError(code, seq)
        return self.out, self.loss


def run_cabi(am, edges, weights, start_end, seq_lens, n_states, out_mode=cabi.OUT_NEG_LOG):
    p = DeviceProblem(am, edges, weights, start_end, seq_lens, n_states)
    out, loss = p.run(out_mode)
    torch.cuda.synchronize()
    return out.cpu().numpy(), loss.cpu().numpy()
