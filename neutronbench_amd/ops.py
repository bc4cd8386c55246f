"""Host-side mirrors of the reference's GPU graph operators: objects with forward()/backward()
that allocate their output like the reference does and call the HIP library through the C ABI.

  ForwardSingleGPUfuseOp   core/ntsSingleGPUFusedGraphOp.hpp:49-70  (full-graph GCN aggregation)
  SingleGPUSampleGraphOp   core/ntsMiniBatchGraphOp.hpp:248-376     (sampled-layer aggregation)
  SingleGPUEdgeSoftMax     core/ntsDistGPUGraphOp.hpp:262-310       (DistGPUEdgeSoftMax kernels)
  SingleGPUScatterSrc/Dst, SingleGPUAggregateDst   core/ntsDistGPUGraphOp.hpp:128-260
  GATAttentionOp, GATAggregateOp   the fused forms of toolkits/GAT_CPU_DIST_OPTM.hpp:186-228
"""
import torch

from .abi import call, ptr
from .stream import CudaStream


def _check2d(t):
    if t.dim() != 2 or t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError("graph operators take 2-D contiguous fp32 tensors (NtsScheduler::getWritableBuffer)")


class ForwardSingleGPUfuseOp:
    """X' = A X on the whole graph: forward gathers by destination over the CSC, backward gathers
    by source over the CSR with edge_weight_backward."""

    def __init__(self, chunk, with_weight=True):
        self.chunk = chunk
        self.with_weight = with_weight

    def _run(self, plan, x, offsets, indices, weight, base):
        _check2d(x)
        out = torch.empty_like(x)
        call("nts_spmm_gather_planned", plan.handle, ptr(x), ptr(out), ptr(weight) if self.with_weight else 0,
             ptr(offsets), ptr(indices), base, x.shape[1], 0, torch.cuda.current_stream(x.device).cuda_stream)
        return out

    def forward(self, f_input):
        c = self.chunk
        return self._run(c.plan_forward, f_input, c.column_offset_gpu, c.row_indices_gpu, c.edge_weight_forward_gpu,
                         c.src_range[0])

    def backward(self, f_output_grad):
        c = self.chunk
        return self._run(c.plan_backward, f_output_grad, c.row_offset_gpu, c.column_indices_gpu,
                         c.edge_weight_backward_gpu, c.dst_range[0])


class SingleGPUSampleGraphOp:
    """Aggregation on one sampled layer; result complete when the call returns (the reference
    synchronises its stream, core/ntsMiniBatchGraphOp.hpp:315, 372)."""

    def __init__(self, subgraphs, layer, cuda_stream=None, sync=True):
        self.sg = subgraphs[layer]
        self.cs = cuda_stream or CudaStream(device=self.sg.dev_column_offset.device)
        self.sync = sync

    def forward(self, f_input):
        _check2d(f_input)
        sg = self.sg
        F = f_input.shape[1]
        out = torch.zeros(sg.v_size, F, dtype=torch.float32, device=f_input.device)
        if 0 < sg.max_in_degree <= 256:
            # the sampler bounded every destination's edges by its fanout: one launch, nothing to cut
            call("nts_spmm_gather_bounded", ptr(f_input), ptr(out), ptr(sg.dev_ewf()), ptr(sg.dev_c_o()),
                 ptr(sg.dev_r_i()), 0, sg.v_size, sg.e_size, F, 1, sg.max_in_degree, self.cs.stream)
        else:
            self.cs.Gather_By_Dst_From_Src(f_input, out, sg.dev_ewf(), sg.dev_r_i(), sg.dev_c_o(), 0, 0, 0, 0,
                                           sg.e_size, sg.v_size, F, True, False)
        if self.sync:
            self.cs.CUDA_DEVICE_SYNCHRONIZE()
        return out

    def backward(self, f_output_grad):
        _check2d(f_output_grad)
        sg = self.sg
        F = f_output_grad.shape[1]
        gin = torch.zeros(sg.src_size, F, dtype=torch.float32, device=f_output_grad.device)
        self.cs.Gather_By_Src_From_Dst(f_output_grad, gin, sg.dev_ewb(), sg.dev_r_o(), sg.dev_c_i(), 0, 0, 0, 0,
                                       sg.e_size, sg.src_size, F, True, False)
        if self.sync:
            self.cs.CUDA_DEVICE_SYNCHRONIZE()
        return gin


class SingleGPUEdgeSoftMax:
    """Per-destination softmax of an [E, H] edge tensor; caches its output for the backward."""

    def __init__(self, column_offset, Vd, cuda_stream=None):
        self.co, self.Vd = column_offset, Vd
        self.cs = cuda_stream or CudaStream(device=column_offset.device)
        self.cached = None

    def forward(self, f_input):
        _check2d(f_input)
        out = torch.empty_like(f_input)
        self.cs.Edge_Softmax_Forward_Block(out, f_input, None, None, self.co, self.Vd, f_input.shape[1])
        self.cached = out
        return out

    def backward(self, f_output_grad):
        _check2d(f_output_grad)
        gin = torch.empty_like(f_output_grad)
        self.cs.Edge_Softmax_Backward_Block(gin, f_output_grad, self.cached, None, self.co, self.Vd,
                                            f_output_grad.shape[1])
        return gin


class SingleGPUScatterSrc:
    """msg[e] = x[src(e)];  backward sums edge gradients per source through the CSR permutation."""

    def __init__(self, layer, cuda_stream=None):
        self.sg = layer
        self.cs = cuda_stream or CudaStream(device=layer.dev_column_offset.device)

    def forward(self, x):
        _check2d(x)
        sg = self.sg
        msg = torch.empty(sg.e_size, x.shape[1], dtype=torch.float32, device=x.device)
        self.cs.Scatter_Src_Mirror_to_Msg(msg, x, sg.dev_r_i(), sg.dev_c_o(), None, sg.v_size, x.shape[1])
        return msg

    def backward(self, g_msg):
        _check2d(g_msg)
        sg = self.sg
        out = torch.zeros(sg.src_size, g_msg.shape[1], dtype=torch.float32, device=g_msg.device)
        self.cs.Gather_Msg_To_Src_Mirror(out, g_msg, sg.dev_r_o(), sg.dev_csr_to_csc, sg.src_size, g_msg.shape[1])
        return out


class SingleGPUScatterDst:
    """msg[e] = x[dst(e)];  backward sums the edge gradients of every destination."""

    def __init__(self, layer, cuda_stream=None):
        self.sg = layer
        self.cs = cuda_stream or CudaStream(device=layer.dev_column_offset.device)

    def forward(self, x):
        _check2d(x)
        sg = self.sg
        msg = torch.empty(sg.e_size, x.shape[1], dtype=torch.float32, device=x.device)
        self.cs.Scatter_Dst_to_Msg(msg, x, sg.dev_r_i(), sg.dev_c_o(), sg.v_size, x.shape[1])
        return msg

    def backward(self, g_msg):
        _check2d(g_msg)
        sg = self.sg
        out = torch.zeros(sg.v_size, g_msg.shape[1], dtype=torch.float32, device=g_msg.device)
        self.cs.Gather_Msg_to_Dst(out, g_msg, sg.dev_r_i(), sg.dev_c_o(), sg.v_size, g_msg.shape[1])
        return out


class SingleGPUAggregateDst:
    """out[d] = sum of the edge rows of d;  backward copies the destination gradient to its edges."""

    def __init__(self, layer, cuda_stream=None):
        self.sg = layer
        self.cs = cuda_stream or CudaStream(device=layer.dev_column_offset.device)

    def forward(self, msg):
        _check2d(msg)
        sg = self.sg
        out = torch.zeros(sg.v_size, msg.shape[1], dtype=torch.float32, device=msg.device)
        self.cs.Gather_Msg_to_Dst(out, msg, sg.dev_r_i(), sg.dev_c_o(), sg.v_size, msg.shape[1])
        return out

    def backward(self, g_out):
        _check2d(g_out)
        sg = self.sg
        g_msg = torch.empty(sg.e_size, g_out.shape[1], dtype=torch.float32, device=g_out.device)
        self.cs.Scatter_Dst_to_Msg(g_msg, g_out, sg.dev_r_i(), sg.dev_c_o(), sg.v_size, g_out.shape[1])
        return g_msg


class GATAttentionOp:
    """alpha = edge_softmax(leaky_relu(el[src] + er[dst])) in one kernel; two-input operator:
    backward returns the gradient of el, get_additional_grad() the gradient of er."""

    def __init__(self, layer, slope=0.2):
        self.sg, self.slope = layer, slope
        self.alpha = self.el = self.er = self.ger = None

    def forward(self, el, er):
        _check2d(el)
        _check2d(er)
        sg = self.sg
        H = el.shape[1]
        alpha = torch.empty(sg.e_size, H, dtype=torch.float32, device=el.device)
        stream = torch.cuda.current_stream(el.device).cuda_stream
        call("nts_gat_attention_fwd_bounded", ptr(alpha), ptr(el), ptr(er), ptr(sg.dev_c_o()), ptr(sg.dev_r_i()),
             sg.v_size, H, self.slope, getattr(sg, "max_in_degree", 0), stream)
        self.alpha, self.el, self.er = alpha, el, er
        return alpha

    def backward(self, g_alpha):
        _check2d(g_alpha)
        sg = self.sg
        H = g_alpha.shape[1]
        dev = g_alpha.device
        stream = torch.cuda.current_stream(dev).cuda_stream
        gs = torch.empty_like(g_alpha)
        self.ger = torch.empty(sg.v_size, H, dtype=torch.float32, device=dev)
        call("nts_gat_attention_bwd_bounded", ptr(gs), ptr(self.ger), ptr(g_alpha), ptr(self.alpha), ptr(self.el),
             ptr(self.er), ptr(sg.dev_c_o()), ptr(sg.dev_r_i()), sg.v_size, H, self.slope,
             getattr(sg, "max_in_degree", 0), stream)
        gel = torch.empty(sg.src_size, H, dtype=torch.float32, device=dev)
        call("nts_gather_edge_to_src", ptr(gel), ptr(gs), ptr(sg.dev_r_o()), ptr(sg.dev_csr_to_csc), sg.src_size, H, 0,
             stream)
        return gel

    def get_additional_grad(self):
        return self.ger


class GATAggregateOp:
    """out[d, h, :] = sum_e alpha[e, h] * x[src(e), h, :]; two-input operator: backward returns the
    gradient of x, get_additional_grad() the gradient of alpha."""

    def __init__(self, layer, heads):
        self.sg, self.H = layer, heads
        self.x = self.alpha = self.galpha = None

    def forward(self, x, alpha):
        _check2d(x)
        _check2d(alpha)
        sg = self.sg
        Fh = x.shape[1] // self.H
        out = torch.empty(sg.v_size, x.shape[1], dtype=torch.float32, device=x.device)
        stream = torch.cuda.current_stream(x.device).cuda_stream
        call("nts_spmm_gather_heads_bounded", ptr(x), ptr(out), ptr(alpha), 0, ptr(sg.dev_c_o()), ptr(sg.dev_r_i()),
             sg.v_size, sg.e_size, self.H, Fh, 0, getattr(sg, "max_in_degree", 0), stream)
        self.x, self.alpha = x, alpha
        return out

    def backward(self, g_out):
        _check2d(g_out)
        sg = self.sg
        Fh = g_out.shape[1] // self.H
        dev = g_out.device
        stream = torch.cuda.current_stream(dev).cuda_stream
        gx = torch.empty(sg.src_size, g_out.shape[1], dtype=torch.float32, device=dev)
        call("nts_spmm_gather_heads", ptr(g_out), ptr(gx), ptr(self.alpha), ptr(sg.dev_csr_to_csc), ptr(sg.dev_r_o()),
             ptr(sg.dev_c_i()), sg.src_size, sg.e_size, self.H, Fh, 0, stream)
        self.galpha = torch.empty(sg.e_size, self.H, dtype=torch.float32, device=dev)
        call("nts_sddmm_heads", ptr(self.galpha), ptr(self.x), ptr(g_out), ptr(sg.dev_c_o()), ptr(sg.dev_r_i()),
             sg.v_size, self.H, Fh, stream)
        return gx

    def get_additional_grad(self):
        return self.galpha
