"""GNN layers over sampled blocks without DGL.

The reference's DP models take their layers from DGL (examples/model.py:38-41);
its own layers (python/npc/model/sageconv.py:118-188 MPSAGEConv, Aggregate
:100-114) do A(XW) with the library's SpMM operator and get the backward pass
from the same operator with the edges reversed.  The layers here keep that
arithmetic on a Block of this package: the forward sum reads the sampler's
fixed-stride layout directly (no atomics), the backward sum runs over the
block's CSR order (edges grouped by source), so both directions are
reproducible.
"""
import torch
from torch import nn

from . import capi


class BlockAggregate(torch.autograd.Function):
    """out[d] = sum (or mean) over the block's edges (s -> d) of X[s]."""

    @staticmethod
    def forward(ctx, block, X, mean):
        ctx.block, ctx.mean = block, mean
        out = capi.spmm_block(block.relabeled, block.num_dst, block.fanout, X.contiguous(), mean=mean)
        return out if X.dtype == torch.float32 else out.to(X.dtype)      # sums are fp32 inside the kernel

    @staticmethod
    def backward(ctx, dZ):
        block = ctx.block
        dZ = dZ.contiguous()
        if ctx.mean:
            indptr = block.csc()[0]
            dZ = dZ / (indptr[1:] - indptr[:-1]).clamp(min=1).to(dZ.dtype)[:, None]
        indptr, dst, eids = block.csr()                # edges grouped by source, by increasing edge id
        src = block.row[eids]
        # every source row is stored whole by the wavefront that holds its edges (or zeroed and added when it
        # spans two): no zero-fill, no atomics for the bulk, sums in edge order
        dX = capi.spmm_heads(dst, src, dZ, None, block.num_src, grouped=True, out_indptr=indptr)
        return None, dX.to(dZ.dtype), None


class SAGEConv(nn.Module):
    """GraphSAGE layer, mean aggregator, with the reference's arithmetic
    (python/npc/model/sageconv.py:118-188): fc_self(h_dst) + fc_neigh(mean of
    the neighbours), the linear map applied before the aggregation when it
    shrinks the features."""

    def __init__(self, in_feats, out_feats, bias=True, activation=None):
        super().__init__()
        self.in_feats, self.out_feats, self.activation = in_feats, out_feats, activation
        self.fc_neigh = nn.Linear(in_feats, out_feats, bias=False)
        self.fc_self = nn.Linear(in_feats, out_feats, bias=bias)
        gain = nn.init.calculate_gain("relu")
        nn.init.xavier_uniform_(self.fc_self.weight, gain=gain)
        nn.init.xavier_uniform_(self.fc_neigh.weight, gain=gain)

    def forward(self, block, feat):
        """feat: [block.num_src, in_feats]; the first num_dst rows are the destinations."""
        h_self = feat[:block.num_dst]
        if self.in_feats > self.out_feats:
            h_neigh = BlockAggregate.apply(block, self.fc_neigh(feat), True)
        else:
            h_neigh = self.fc_neigh(BlockAggregate.apply(block, feat, True))
        rst = self.fc_self(h_self) + h_neigh
        return self.activation(rst) if self.activation is not None else rst


class GraphConv(nn.Module):
    """GCN layer with the reference's arithmetic (python/npc/model/graphconv.py:
    159-232, MPGraphConv): the fanout stands in for the degrees in the
    normalisation ("both": fanout^-1/2 on either side, "left"/"right": 1/fanout
    on one), the weight is applied before the sum."""

    def __init__(self, in_feats, out_feats, norm="both", bias=True, activation=None):
        super().__init__()
        if norm not in ("none", "both", "right", "left"):
            raise KeyError(f'Invalid norm value. Must be either "none", "both", "right" or "left". But got "{norm}".')
        self.norm, self.activation = norm, activation
        self.weight = nn.Parameter(torch.empty(in_feats, out_feats))
        self.bias = nn.Parameter(torch.zeros(out_feats)) if bias else None
        nn.init.xavier_uniform_(self.weight)

    def forward(self, block, feat):
        fanout = float(block.fanout)
        if self.norm in ("left", "both"):
            feat = feat * (fanout ** -0.5 if self.norm == "both" else 1.0 / fanout)
        rst = BlockAggregate.apply(block, torch.matmul(feat, self.weight), False)
        if self.norm in ("right", "both"):
            rst = rst * (fanout ** -0.5 if self.norm == "both" else 1.0 / fanout)
        if self.bias is not None:
            rst = rst + self.bias
        return self.activation(rst) if self.activation is not None else rst


class GATAggregate(torch.autograd.Function):
    """out[d, h] = sum over the block's edges (s -> d) of softmax_d(LeakyReLU(el[s, h] + er[d, h])) * ft[s, h]
    (python/npc/model/gatconv.py:118-126), forward and backward fused over the
    block: forward = one kernel from the fixed-stride layout; backward = one
    kernel per (destination, head) for the logit gradients, then the two sums
    over the edges of a source on the block's CSR order."""

    @staticmethod
    def forward(ctx, block, ft, el, er, negative_slope):
        ft, el, er = ft.contiguous(), el.contiguous().float(), er.contiguous().float()
        out, attn = capi.gat_block(block.relabeled, block.num_dst, block.fanout, ft, el, er, negative_slope,
                                   want_attn=True)
        ctx.block, ctx.slope = block, negative_slope
        ctx.save_for_backward(ft, el, er, attn)
        return out.to(ft.dtype) if ft.dtype != torch.float32 else out

    @staticmethod
    def backward(ctx, d_out):
        block = ctx.block
        ft, el, er, attn = ctx.saved_tensors
        d_out = d_out.contiguous().float()
        csc_indptr = block.csc()[0]
        indptr, dst, eids = block.csr()
        E = eids.numel()
        a_edge, dz_edge, d_er = capi.gat_block_backward(block.relabeled, block.num_dst, block.fanout, ft, el, er,
                                                        ctx.slope, attn, d_out, csc_indptr, E)
        # sums over the edges of a source, in the block's CSR order; the per-edge weights stay in COO order
        src = block.row[eids]
        d_ft, d_el = capi.spmm_heads(dst, src, d_out, a_edge, block.num_src, weight_row=eids, grouped=True,
                                     head_weights2=dz_edge, out_indptr=indptr)
        return None, d_ft.to(ft.dtype), d_el, d_er, None


class GATConv(nn.Module):
    """GAT layer (python/npc/model/gatconv.py:207-236: fc, attention logits,
    LeakyReLU, edge softmax, weighted sum, bias).  Under torch.no_grad() the
    logits come from the library's kernel too; otherwise from torch, so that
    autograd carries them, and the aggregation is GATAggregate."""

    def __init__(self, in_feats, out_feats, num_heads, negative_slope=0.2, bias=True, activation=None):
        super().__init__()
        self.num_heads, self.out_feats, self.negative_slope, self.activation = (num_heads, out_feats,
                                                                                negative_slope, activation)
        self.fc = nn.Linear(in_feats, out_feats * num_heads, bias=False)
        self.attn_l = nn.Parameter(torch.empty(num_heads, out_feats))
        self.attn_r = nn.Parameter(torch.empty(num_heads, out_feats))
        self.bias = nn.Parameter(torch.zeros(num_heads * out_feats)) if bias else None
        gain = nn.init.calculate_gain("relu")
        nn.init.xavier_normal_(self.fc.weight, gain=gain)
        nn.init.xavier_normal_(self.attn_l, gain=gain)
        nn.init.xavier_normal_(self.attn_r, gain=gain)

    def forward(self, block, feat):
        ft = self.fc(feat).view(block.num_src, self.num_heads, self.out_feats).contiguous()
        if torch.is_grad_enabled() and (ft.requires_grad or self.attn_l.requires_grad):
            el = (ft * self.attn_l).sum(-1)
            er = (ft[:block.num_dst] * self.attn_r).sum(-1)
            rst = GATAggregate.apply(block, ft, el, er, self.negative_slope)
        else:
            el = capi.gat_scores(ft, self.attn_l.detach().float().contiguous())
            er = capi.gat_scores(ft[:block.num_dst].contiguous(), self.attn_r.detach().float().contiguous())
            rst = capi.gat_block(block.relabeled, block.num_dst, block.fanout, ft, el, er, self.negative_slope)
        if self.bias is not None:
            rst = rst + self.bias.view(1, self.num_heads, self.out_feats)
        return self.activation(rst) if self.activation is not None else rst
