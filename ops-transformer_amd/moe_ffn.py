"""The quantized MoE expert FFN as a chain of the four aclnn operators (the caller side of the path).

    aclnnMoeInitRoutingV2 -> aclnnGroupedMatmulSwigluQuant -> aclnnGroupedMatmulV4 -> aclnnMoeFinalizeRoutingV2

The reference has no in-repo code that chains them; real callers (torch_npu, vLLM-Ascend) do what ``forward`` does.
Glue between the operators:
  * activations arrive already quantized per token (int8 rows + fp32 scale); MoeInitRoutingV2 routes the int8 rows
    (INT8 x is this build's extension: a row gather commutes with per-row quantization bit-exactly) and a second
    MoeInitRoutingV2 call routes the [T, 1] column of per-token scales the same way;
  * routing emits the int32 cumsum (expertTokensCountOrCumsumFlag 1), which both GEMM operators take as groupList (the
    reference wants int64 there; int32 is accepted as an extension, so no cast kernel sits between the operators);
  * MoeFinalizeRoutingV2 is called with dropPadMode 2 because V2's index is the row arrangement
    expandedRowIdx[n*K + k] = destination.
``routing="v3"`` puts aclnnMoeInitRoutingV3 at the head instead: one call (quantMode -1) routes the rows and carries
the per-token scales along as expandedScale, and emits the int64 cumsum (expertTokensNumType 0); scatter-type index
(rowIdxType 1).
``fused_combine=True`` replaces the last two operators by aclnnGroupedMatmulFinalizeRoutingV3 (down projection with
the weighted combine as scatter-add): routing then emits the gather-type index (rowIdxType 0), from which the glue
derives the fused operator's rowIndex (destination token = source // K) and logit (the top-k weight of that source);
the result is fp32 [T, H], and the order of the K additions per token is not fixed.
"""
import torch

from . import aclnn


class MoeFfnW8A8:
    """Expert weights resident on one GPU plus preallocated intermediates for a fixed (tokens, top_k).

    w13: int8 storage [E, 2I, H]  (gate/up projection, K-contiguous: row n holds the H weights of output channel n;
         channels [0, I) are the activated half, [I, 2I) the linear half)
    w13_scale: fp32 [E, 2I]
    w2:  int8 storage [E, H, I]   (down projection, K-contiguous)
    w2_scale:  fp32 or bf16 [E, H]
    The operators see the reference layout [E, K, N] through transposed views of this storage.
    """

    def __init__(self, w13, w13_scale, w2, w2_scale, out_dtype=torch.bfloat16, routing="v2", fused_combine=False,
                 weight_nz=False, weight_row_major=False):
        assert routing in ("v2", "v3")
        assert not (fused_combine and routing != "v3")
        assert not (fused_combine and weight_nz)
        assert not (weight_nz and weight_row_major)
        self.routing = routing
        self.fused_combine = fused_combine
        # weight_nz: hand the operators the reference's FRACTAL_NZ weights ([E, N/32, K/16, 16, 32]) instead of the
        # transposed views; the blocked copies are made here, once
        self.w13_nz = self.to_nz(w13) if weight_nz else None
        self.w2_nz = self.to_nz(w2) if weight_nz else None
        assert w13.dtype == torch.int8 and w2.dtype == torch.int8
        self.w13_view = w13.transpose(1, 2)  # [E, H, 2I]
        self.w2_view = w2.transpose(1, 2)    # [E, I, H]
        if weight_row_major:
            # the reference's plain ND layout: contiguous [E, K, N] copies, made here, once
            self.w13_view = self.w13_view.contiguous()
            self.w2_view = self.w2_view.contiguous()
        self.w13_scale = w13_scale
        self.w2_scale = w2_scale
        self.num_experts = w13.shape[0]
        self.hidden = w13.shape[2]
        self.inter = w13.shape[1] // 2
        self.out_dtype = out_dtype
        self.device = w13.device
        self._buf_key = None

    @staticmethod
    def to_nz(w_enk):
        """K-contiguous storage [E, N, K] -> blocked [E, N/32, K/16, 16, 32] (element (k, n) at [n/32][k/16][k%16][n%32])."""
        E, N, K = w_enk.shape
        return w_enk.view(E, N // 32, 32, K // 16, 16).permute(0, 1, 3, 4, 2).contiguous()

    def _buffers(self, T, K):
        if self._buf_key == (T, K):
            return
        dev, M, H, I, E = self.device, T * K, self.hidden, self.inter, self.num_experts
        self.expanded_x = torch.empty((M, H), dtype=torch.int8, device=dev)
        self.expanded_row_idx = torch.empty((M,), dtype=torch.int32, device=dev)
        self.cumsum = torch.empty((E,), dtype=torch.int64 if self.routing == "v3" else torch.int32, device=dev)
        self.expanded_scale = torch.empty((M,), dtype=torch.float32, device=dev)
        self.row_idx_scratch = torch.empty((M,), dtype=torch.int32, device=dev)
        self.h = torch.empty((M, I), dtype=torch.int8, device=dev)
        self.h_scale = torch.empty((M,), dtype=torch.float32, device=dev)
        self.y = torch.empty((M, H), dtype=self.out_dtype, device=dev)
        self.out = torch.empty((T, H), dtype=torch.float32 if self.fused_combine else self.out_dtype, device=dev)
        # one workspace shared by the chain; it grows to the largest phase-1 request on the first pass
        self.workspace = aclnn.Workspace()
        self._buf_key = (T, K)

    def forward(self, xq, x_scale, topk_idx, topk_weight):
        """xq int8 [T, H]; x_scale fp32 [T]; topk_idx int32 [T, K]; topk_weight fp32/bf16 [T, K] -> out [T, H]."""
        T, K = topk_idx.shape
        self._buffers(T, K)
        E = self.num_experts
        if self.routing == "v3":
            aclnn.moe_init_routing_v3(xq, topk_idx, x_scale, expert_num=E, expert_tokens_num_type=0, quant_mode=-1,
                                      row_idx_type=0 if self.fused_combine else 1,
                                      out=(self.expanded_x, self.expanded_row_idx, self.cumsum, self.expanded_scale),
                                      workspace=self.workspace)
        else:
            aclnn.moe_init_routing_v2(xq, topk_idx, 0, 0, E, 0, 1, False,
                                      out=(self.expanded_x, self.expanded_row_idx, self.cumsum, None),
                                      workspace=self.workspace)
            aclnn.moe_init_routing_v2(x_scale.view(T, 1), topk_idx, 0, 0, E, 0, 0, False,
                                      out=(self.expanded_scale.view(T * K, 1), self.row_idx_scratch, None, None),
                                      workspace=self.workspace)
        aclnn.grouped_matmul_swiglu_quant(self.expanded_x, None if self.w13_nz is not None else self.w13_view, self.cumsum,
                                          self.w13_scale, self.expanded_scale, out=(self.h, self.h_scale),
                                          weight_nz=None if self.w13_nz is None else (self.w13_nz, "nz5d"),
                                          workspace=self.workspace)
        if self.fused_combine:
            source = self.expanded_row_idx.long()                       # expanded row -> flat (token, k) position
            logit = topk_weight.reshape(-1).float()[source]
            aclnn.grouped_matmul_finalize_routing(self.h, self.w2_view, self.w2_scale, source // K, T, self.cumsum,
                                                  group_list_type=0, per_token_scale=self.h_scale, logit=logit,
                                                  out=self.out, workspace=self.workspace)
            return self.out
        aclnn.grouped_matmul_v4([self.h], None if self.w2_nz is not None else [self.w2_view],
                                weight_nz=None if self.w2_nz is None else (self.w2_nz, "nz5d"),
                                scale=[self.w2_scale], per_token_scale=[self.h_scale],
                                group_list=self.cumsum, split_item=3, group_type=0, group_list_type=0, act_type=0,
                                out=[self.y], workspace=self.workspace)
        aclnn.moe_finalize_routing_v2(self.y, self.expanded_row_idx, scales=topk_weight, drop_pad_mode=2, out=self.out)
        return self.out

    def capture(self, xq, x_scale, topk_idx, topk_weight):
        """Records one pass over these input buffers into a HIP graph and returns (graph, out).

        ``graph.replay()`` re-runs the recorded kernels on whatever the four input buffers hold at that time (same
        shapes, same addresses) and leaves the result in ``out``.  The first phases (validation, planning) ran once,
        at capture time: a replay is the second phases only, enqueued with a single launch.  One eager pass comes
        first so that buffers, the workspace and kernel attributes exist before recording starts; nothing in the second
        phases allocates, synchronises or clears memory with a memset node."""
        self.forward(xq, x_scale, topk_idx, topk_weight)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = self.forward(xq, x_scale, topk_idx, topk_weight)
        return graph, out
