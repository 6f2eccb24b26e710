"""Kernel programs: ordered launch lists for one quantized linear and for one MoE expert layer.

The engine runs a *program* -- an ordered list of kernel records whose buffers it owns
(crates/orinfer-engine/src/backend/cuda/executor.rs:1095-1124).  These classes are that list for
the paths of this library, with every buffer allocated once up front (torch is used only for
device memory and the stream), so `run()` only enqueues and can be captured in a graph.
Program order of the expert layer follows python/orinfer_build/models/flash_next (router top-k,
histogram, offsets, tiles, A8, dispatch, grouped gate_up, SwiGLU->A8, grouped down, combine).
"""
import numpy as np
import torch

from . import codebook
from .lib import ORX_ERR_BAD_VARIANT, Kernel, OrxError


def _dev(array):
    a = np.ascontiguousarray(array)
    view = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32}.get(a.dtype)
    return torch.from_numpy(a.view(view) if view else a).cuda()


class QuantizedLinear:
    """A8 quantiser + one projection (E8P-Q4 or W8A8) with a dynamic row count up to `capacity`."""

    def __init__(self, codec, weight, scales, capacity, *, packed_k=0, algorithm="auto", block_m=0, book=None):
        if codec not in ("q4", "w8"):
            raise ValueError("codec must be q4 or w8")
        self.codec, self.capacity = codec, capacity
        scales = np.asarray(scales)
        self.n = scales.shape[0]
        weight = np.asarray(weight)
        if codec == "q4":
            self.k = weight.shape[1] * 8
            stored = codebook.q4_to_k_major(weight, 128) if packed_k == 128 else weight
        else:
            self.k = weight.shape[1]
            stored = weight
        self.weight = _dev(stored)
        self.scales = _dev(scales)
        self.book = _dev(codebook.book() if book is None else book)
        self.a_q = torch.empty((capacity, self.k), dtype=torch.int8, device="cuda")
        self.a_s = torch.empty((capacity, 1), dtype=torch.float16, device="cuda")
        self.out = torch.empty((capacity, self.n), dtype=torch.float16, device="cuda")
        self.quantizer = Kernel("activation_quantization", K=self.k)
        # workspace=True: the projection takes a `Workspace` buffer (allocated below, once, at the size
        # orx_workspace_bytes reports) for split tiles and decode-once launches
        variant = dict(M=capacity, N=self.n, K=self.k, dynamic_rows=True, algorithm=algorithm, workspace=True)
        if block_m:
            variant["block_m"] = block_m
        if codec == "q4":
            if packed_k:
                variant["packed_k"] = packed_k
            self.projection = Kernel("e8p_q4_projection", **variant)
        else:
            self.projection = Kernel("int8_projection", **variant)
        self.workspace = self.projection.workspace()

    def quantize(self, x16, stream=None):
        rows = x16.shape[0]
        self.quantizer(stream=stream, Mask=None, Q=self.a_q, S=self.a_s, X=x16, rows=rows)
        return rows

    def project(self, rows, stream=None):
        if self.codec == "q4":
            self.projection(stream=stream, A=self.a_q, AS=self.a_s, Book=self.book, Out=self.out, S=self.scales,
                            W=self.weight, Workspace=self.workspace, m=rows)
        else:
            self.projection(stream=stream, A=self.a_q, Output=self.out, TokenScale=self.a_s, Weight=self.weight,
                            WeightScale=self.scales, Workspace=self.workspace, m=rows)
        return self.out[:rows]

    def run(self, x16, stream=None):
        return self.project(self.quantize(x16, stream), stream)


class MoeLayer:
    """Q2A8 expert layer: token-sort, grouped gate_up, SwiGLU->A8, grouped down, weighted combine."""

    def __init__(self, tokens, experts, top_k, hidden, intermediate, gate_up, gate_up_scales, down, down_scales,
                 block_m=32, packed_k=128, fused_metadata=None, fused_dispatch=True, signs=None, fused_stages=None,
                 keep_intermediates=False, grouped_algorithm="auto"):
        self.tokens, self.experts, self.top_k = tokens, experts, top_k
        self.hidden, self.inter, self.block_m = hidden, intermediate, block_m
        assignments = tokens * top_k
        self.assignments = assignments
        # capacity bound of the tile list (kernels/cuda/model/moe.py:263-264)
        self.tile_capacity = (assignments + block_m - 1) // block_m + min(experts, assignments)
        gate_up, down = np.asarray(gate_up), np.asarray(down)
        if packed_k == 128:
            gate_up, down = codebook.q2_to_k_major(gate_up), codebook.q2_to_k_major(down)
        self.w1, self.w2 = _dev(gate_up), _dev(down)
        self.s1, self.s2 = _dev(gate_up_scales), _dev(down_scales)
        self.book = _dev(codebook.book())
        i32 = dict(dtype=torch.int32, device="cuda")
        f16 = dict(dtype=torch.float16, device="cuda")
        i8 = dict(dtype=torch.int8, device="cuda")
        self.ids = torch.empty((tokens, top_k), **i32)
        self.prob = torch.empty((tokens, top_k), dtype=torch.float32, device="cuda")
        self.counts = torch.empty(experts, **i32)
        self.relative = torch.empty((tokens, top_k), **i32)
        self.row_offsets = torch.empty(experts, **i32)
        self.tile_offsets = torch.empty(experts, **i32)
        self.tile_count = torch.empty(1, **i32)
        self.tile_expert = torch.empty(self.tile_capacity, **i32)
        self.tile_row = torch.empty(self.tile_capacity, **i32)
        self.slot_map = torch.empty((tokens, top_k), **i32)
        self.a_q = torch.empty((tokens, hidden), **i8)
        self.a_s = torch.empty((tokens, 1), **f16)
        self.d = torch.empty((assignments, hidden), **i8)
        self.ds = torch.empty((assignments, 1), **f16)
        self.gate_up_out = torch.empty((assignments, 2 * intermediate), **f16)
        self.h_q = torch.empty((assignments, intermediate), **i8)
        self.h_s = torch.empty((assignments, 1), **f16)
        self.down_out = torch.empty((assignments, hidden), **f16)
        self.out = torch.empty((tokens, hidden), **f16)
        common = dict(M=tokens, E=experts, top_k=top_k)
        # one launch for all routing metadata where the fused kernel applies (kernels/cuda/model/moe.py:713-764),
        # the three-kernel form otherwise
        if fused_metadata is None:
            fused_metadata = experts <= 1024 and (16 * experts + 32 + 2 * tokens * top_k) * 4 <= 160 * 1024
        self.k_metadata = Kernel("route_metadata", block_m=block_m, **common) if fused_metadata else None
        self.k_router = Kernel("router_topk", renormalize=True, **common)
        self.k_histogram = Kernel("expert_histogram", **common)
        self.k_offsets = Kernel("expert_offsets", E=experts, block_m=block_m)
        self.k_tiles = Kernel("expert_tiles", block_m=block_m, **common)
        # the dispatch quantises the fp16 rows on its way (one launch instead of quantiser + copy) where
        # the row layout allows it
        self.fused_dispatch = fused_dispatch and hidden % 8 == 0
        self.k_a8 = Kernel("activation_quantization", K=hidden)
        self.k_dispatch = Kernel("expert_dispatch", H=hidden, scale_group=hidden, **common,
                                 **({"input_dtype": "float16"} if self.fused_dispatch else {}))
        # signs: the layer's input is rotated first (block-128 signed Hadamard); rotation, A8 and the
        # scatter to the expert-sorted slots are one launch (kernels/cuda/model/rotation_a8.py:558-604)
        self.signs = None if signs is None else _dev(np.asarray(signs, np.int8))
        self.k_rotate_dispatch = None
        if signs is not None:
            self.k_rotate_dispatch = Kernel("rotate_expert_a8", M=tokens, K=hidden, routing="scatter", top_k=top_k,
                                            experts=experts, hand_over="int8")
        grouped = dict(rows=assignments, E=experts, tiles=self.tile_capacity, block_m=block_m, packed_k=packed_k,
                       algorithm=grouped_algorithm)
        self.k_gate_up = Kernel("e8p_decode_grouped", N=2 * intermediate, K=hidden, **grouped)
        self.k_swiglu_a8 = Kernel("activation_quantization", K=intermediate, fused=True)
        self.k_down = Kernel("e8p_decode_grouped", N=hidden, K=intermediate, **grouped)
        # Five launches instead of seven where the resident expert kernel takes the shapes:
        #   router top-k that also quantises every token's row (once per token, not once per route),
        #   metadata that also writes SlotMap, its inverse and zeroed per-slot maxima,
        #   gate_up that gathers the int8 token rows by slot while it stages a tile (no dispatch copy) and
        #     whose epilogue writes fp16(silu(gate) * up) and raises every slot's largest magnitude,
        #   down that quantises those fp16 rows while it stages a tile (no SwiGLU->A8 launch),
        #   combine.
        # The library refuses the variants it does not serve that way, and the seven-launch program stays.
        self.fused_stages = False
        self.keep_intermediates = keep_intermediates
        if fused_stages is not False and fused_metadata and signs is None and hidden % 8 == 0:
            try:
                self.k_router_a8 = Kernel("router_topk", renormalize=True, quantize_hidden=hidden, **common)
                self.k_metadata_slots = Kernel("route_metadata", block_m=block_m, slot_maps=True, **common)
                self.k_gate_up_fused = Kernel("e8p_decode_grouped", N=2 * intermediate, K=hidden, gather=True,
                                              epilogue="swiglu", **grouped)
                self.k_down_fused = Kernel("e8p_decode_grouped", N=hidden, K=intermediate, input_dtype="float16",
                                           **grouped)
                self.slot_token = torch.empty(assignments, **i32)
                self.row_max = torch.empty(assignments, **i32)
                self.act = torch.empty((assignments, intermediate), **f16)
                self.fused_stages = True
            except OrxError as error:
                if fused_stages or error.code != ORX_ERR_BAD_VARIANT:
                    raise
        self.k_combine = Kernel("moe_combine", H=hidden, slots=assignments, **common)

    def run(self, x16, logits, stream=None):
        s = stream
        if self.fused_stages:
            return self._run_fused(x16, logits, s)
        self.k_router(stream=s, IDs=self.ids, Logits=logits, Prob=self.prob)
        if self.k_metadata is not None:
            self.k_metadata(stream=s, Counts=self.counts, IDs=self.ids, RelativeSlot=self.relative,
                            RowOffsets=self.row_offsets, TileCount=self.tile_count, TileExpert=self.tile_expert,
                            TileOffsets=self.tile_offsets, TileRow=self.tile_row)
        else:
            self.k_histogram(stream=s, Counts=self.counts, IDs=self.ids, RelativeSlot=self.relative)
            self.k_offsets(stream=s, Counts=self.counts, RowOffsets=self.row_offsets, TileCount=self.tile_count,
                           TileOffsets=self.tile_offsets)
            self.k_tiles(stream=s, Counts=self.counts, TileExpert=self.tile_expert, TileOffsets=self.tile_offsets,
                         TileRow=self.tile_row)
        if self.k_rotate_dispatch is not None:
            self.k_rotate_dispatch(stream=s, D=self.d, DS=self.ds, IDs=self.ids, Q=None, RelativeSlot=self.relative,
                                   RowOffsets=self.row_offsets, S=self.a_s, Signs=self.signs, SlotMap=self.slot_map,
                                   Sum=None, X=x16)
        elif self.fused_dispatch:
            self.k_dispatch(stream=s, A=x16, D=self.d, DS=self.ds, IDs=self.ids, RelativeSlot=self.relative,
                            RowOffsets=self.row_offsets, Scale=None, SlotMap=self.slot_map)
        else:
            self.k_a8(stream=s, Mask=None, Q=self.a_q, S=self.a_s, X=x16, rows=self.tokens)
            self.k_dispatch(stream=s, A=self.a_q, D=self.d, DS=self.ds, IDs=self.ids, RelativeSlot=self.relative,
                            RowOffsets=self.row_offsets, Scale=self.a_s, SlotMap=self.slot_map)
        routed = dict(Book=self.book, Counts=self.counts, Offsets=self.row_offsets, TileCount=self.tile_count,
                      TileExpert=self.tile_expert, TileRow=self.tile_row)
        self.k_gate_up(stream=s, A=self.d, AS=self.ds, C=self.gate_up_out, P=self.w1, WS=self.s1, **routed)
        self.k_swiglu_a8(stream=s, Mask=None, Q=self.h_q, S=self.h_s, X=self.gate_up_out, rows=self.assignments)
        self.k_down(stream=s, A=self.h_q, AS=self.h_s, C=self.down_out, P=self.w2, WS=self.s2, **routed)
        self.k_combine(stream=s, Expert=self.down_out, Output=self.out, Prob=self.prob, Shared=None, SharedGate=None,
                       SlotMap=self.slot_map)
        return self.out


    def _run_fused(self, x16, logits, s):
        keep = self.keep_intermediates
        self.k_router_a8(stream=s, IDs=self.ids, Logits=logits, Prob=self.prob, Q=self.a_q, S=self.a_s, X=x16)
        self.k_metadata_slots(stream=s, Counts=self.counts, IDs=self.ids, RelativeSlot=self.relative, RowMax=self.row_max,
                              RowOffsets=self.row_offsets, SlotMap=self.slot_map, SlotToken=self.slot_token,
                              TileCount=self.tile_count, TileExpert=self.tile_expert, TileOffsets=self.tile_offsets,
                              TileRow=self.tile_row)
        routed = dict(Book=self.book, Counts=self.counts, Offsets=self.row_offsets, TileCount=self.tile_count,
                      TileExpert=self.tile_expert, TileRow=self.tile_row)
        self.k_gate_up_fused(stream=s, A=self.a_q, AS=self.a_s, Act=self.act, C=self.gate_up_out if keep else None,
                             P=self.w1, RowMax=self.row_max, SlotToken=self.slot_token, WS=self.s1, **routed)
        self.k_down_fused(stream=s, A=self.act, AS=self.h_s if keep else None, C=self.down_out, P=self.w2,
                          Q=self.h_q if keep else None, RowMax=self.row_max, WS=self.s2, **routed)
        self.k_combine(stream=s, Expert=self.down_out, Output=self.out, Prob=self.prob, Shared=None, SharedGate=None,
                       SlotMap=self.slot_map)
        return self.out


class MoeTokenLayer:
    """The same expert layer for ONE token: its routes index the expert banks directly
    (kernels/cuda/model/integer_vq.py:380-444), so there is no sorting, no tile list and no dispatch copy:
    router top-k, gate/up of every route from the shared row (quantised on the way), SwiGLU->A8 per route,
    down per route, weighted combine."""

    def __init__(self, experts, top_k, hidden, intermediate, gate_up, gate_up_scales, down, down_scales, fused=None):
        self.experts, self.top_k, self.hidden, self.inter = experts, top_k, hidden, intermediate
        self.w1 = _dev(codebook.q2_to_k_major(np.asarray(gate_up)))
        self.w2 = _dev(codebook.q2_to_k_major(np.asarray(down)))
        self.s1, self.s2 = _dev(gate_up_scales), _dev(down_scales)
        self.book = _dev(codebook.raw_book())
        f16 = dict(dtype=torch.float16, device="cuda")
        i8 = dict(dtype=torch.int8, device="cuda")
        self.ids = torch.empty((1, top_k), dtype=torch.int32, device="cuda")
        self.prob = torch.empty((1, top_k), dtype=torch.float32, device="cuda")
        self.a_s = torch.empty((1, 1), **f16)
        self.gate_up_out = torch.empty((top_k, 2 * intermediate), **f16)
        self.h_q = torch.empty((top_k, intermediate), **i8)
        self.h_s = torch.empty((top_k, 1), **f16)
        self.down_out = torch.empty((top_k, hidden), **f16)
        self.slot_map = torch.arange(top_k, dtype=torch.int32, device="cuda").view(1, top_k)  # route r is slot r
        self.out = torch.empty((1, hidden), **f16)
        common = dict(M=1, E=experts, top_k=top_k)
        self.k_router = Kernel("router_topk", renormalize=True, **common)
        # gate/up quantises the shared fp16 row itself (no launch for the A8 of one row)
        self.k_gate_up = Kernel("integer_e8p_gemv", E=experts, routes=top_k, N=2 * intermediate, K=hidden,
                                shared_input=True, input_dtype="float16")
        self.k_swiglu_a8 = Kernel("activation_quantization", K=intermediate, fused=True)
        self.k_down = Kernel("integer_e8p_gemv", E=experts, routes=top_k, N=hidden, K=intermediate, shared_input=False)
        self.k_combine = Kernel("moe_combine", H=hidden, slots=top_k, **common)
        # Three launches instead of five where the library has the forms (up to 512 experts): gate/up selects
        # the token's routes itself while it builds its tables (no router launch), down turns the fp16 gate|up
        # rows into SwiGLU -> A8 codes on their way into LDS (no launch in between).
        self.fused = False
        if fused is not False:
            try:
                routes = dict(E=experts, routes=top_k)
                self.k_gate_up_routing = Kernel("integer_e8p_gemv", N=2 * intermediate, K=hidden, shared_input=True,
                                                input_dtype="float16", route_logits=True, renormalize=True, **routes)
                self.k_down_swiglu = Kernel("integer_e8p_gemv", N=hidden, K=intermediate, shared_input=False,
                                            input_dtype="float16", fused_swiglu=True, **routes)
                self.fused = True
            except OrxError as error:
                if fused or error.code != ORX_ERR_BAD_VARIANT:
                    raise

    def run(self, x16, logits, stream=None):
        s = stream
        if self.fused:
            self.k_gate_up_routing(stream=s, A=x16, AS=self.a_s, Book=self.book, C=self.gate_up_out, IDs=self.ids,
                                   Logits=logits, P=self.w1, Prob=self.prob, WS=self.s1)
            self.k_down_swiglu(stream=s, A=self.gate_up_out, AS=self.h_s, Book=self.book, C=self.down_out, IDs=self.ids,
                               P=self.w2, WS=self.s2)
            self.k_combine(stream=s, Expert=self.down_out, Output=self.out, Prob=self.prob, Shared=None, SharedGate=None,
                           SlotMap=self.slot_map)
            return self.out
        self.k_router(stream=s, IDs=self.ids, Logits=logits, Prob=self.prob)
        self.k_gate_up(stream=s, A=x16, AS=self.a_s, Book=self.book, C=self.gate_up_out, IDs=self.ids, P=self.w1,
                       WS=self.s1)
        self.k_swiglu_a8(stream=s, Mask=None, Q=self.h_q, S=self.h_s, X=self.gate_up_out, rows=self.top_k)
        self.k_down(stream=s, A=self.h_q, AS=self.h_s, Book=self.book, C=self.down_out, IDs=self.ids, P=self.w2,
                    WS=self.s2)
        self.k_combine(stream=s, Expert=self.down_out, Output=self.out, Prob=self.prob, Shared=None, SharedGate=None,
                       SlotMap=self.slot_map)
        return self.out
