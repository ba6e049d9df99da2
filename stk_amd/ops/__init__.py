from stk_amd.ops.linear_ops import dds, dsd, sdd, sdd_fused
from stk_amd.ops.matrix_ops import ones_like, row_indices, sum, to_dense, to_sparse
from stk_amd.ops.eltwise_ops import mul
from stk_amd.ops.topology_ops import dmoe_topology
from stk_amd.ops.routing_ops import Route, dsd_scatter, gather_sdd, padded_gather, padded_scatter, route, route_capacity
