"""A partitioned MoE dispatch pipeline over three HIP streams (routing, row movement, exchange): the call pattern Lancet's partition pass
emits for one MoE layer (src/pass/dist_optimization/partition_exprs.cc:1709-1795), on one GPU.

The token batch is cut into P partitions.  Partition i is encoded with the used capacity of partition
i-1 chained in and capacity_factor x P (`:1750-1762`), scheduled at pipeline index i (`:1775`); its
exchange then overlaps the encode of partition i+1.  The chain only links the routing halves of the
encodes (selection + position scan: small, latency-bound kernels), so those run ahead on a stream of
their own while the row movement of earlier partitions streams.  With one GPU there is no all-to-all, so the
exchange stage does what the all-to-allv does to the buffer on either side of the wire: the rows each
expert uses are packed back to back, keyed by elements_per_expert (the send counts,
src/op/dialect/nccl/nccl.cc:373-421), and unpacked into a zero-filled [E, C, M] receive buffer.  The
expert computation is the identity.  Partition i is then decoded from its own receive buffer.

`run_routed_once` is the same layer with the partitions taken as token ranges of ONE routing of the whole batch
(the chained partition encodes, merged, are that routing): one send and one receive buffer shared by the
partitions, every partition scattering, exchanging (at the row ranges it owns) and decoding its own tokens.  It
moves each row once per stage and needs no per-partition buffers.

Streams carry the default priority.  Every buffer is allocated once, in the constructor; `run` only
launches kernels and records events, so it can be called in a loop.
"""
import torch

from . import ops


class PartitionedMoeLayer:
    def __init__(self, S, M, E, n_partitions, capacity_factor=1.0, dtype=torch.float32, gate_is_logits=False,
                 device="cuda"):
        if S % n_partitions != 0:
            raise ValueError("the token count must divide into n_partitions")
        self.S, self.M, self.E, self.P = S, M, E, n_partitions
        self.Sp = S // n_partitions
        self.cf = float(capacity_factor) * n_partitions   # partition_exprs.cc:1754-1760
        self.gate_is_logits = gate_is_logits
        self.C = ops.moe_capacity(self.Sp, E, self.cf)
        dev = torch.device(device)
        P, Sp, C = self.P, self.Sp, self.C
        self.enc = [(torch.empty(Sp, dtype=torch.float32, device=dev),
                     torch.empty((2, Sp), dtype=torch.int32, device=dev),
                     torch.empty(E, dtype=torch.int32, device=dev),
                     torch.empty(E, dtype=torch.int64, device=dev),
                     torch.empty((E, C, M), dtype=dtype, device=dev)) for _ in range(P)]
        # one scan workspace per partition: encodes of neighbouring partitions never share one; they are set up
        # on the current stream and used on the routing / compute streams, hence the synchronisation
        with torch.cuda.device(dev):
            self.ws = [ops.ScanWorkspace(ops.moe_encode_workspace_bytes(Sp, E, 1), dev) for _ in range(P)]
            torch.cuda.current_stream().synchronize()
        self.wire = [torch.empty(E * C * M, dtype=dtype, device=dev) for _ in range(P)]
        self.recv = [torch.empty((E, C, M), dtype=dtype, device=dev) for _ in range(P)]
        self.out = torch.empty((S, M), dtype=dtype, device=dev)
        self.zero_used = torch.zeros(E, dtype=torch.int32, device=dev)
        self.routing = torch.cuda.Stream(device=dev)
        self.compute = torch.cuda.Stream(device=dev)
        self.exchange = torch.cuda.Stream(device=dev)
        self.once = RoutedOnceMoeLayer(S, M, E, n_partitions, capacity_factor, 1, dtype, gate_is_logits, device,
                                       streams=(self.routing, self.compute, self.exchange))
        self.routed = [torch.cuda.Event() for _ in range(P)]
        self.encoded = [torch.cuda.Event() for _ in range(P)]
        self.received = [torch.cuda.Event() for _ in range(P)]

    # ---- the three stages of one partition ----------------------------------------------------
    def _encode(self, i, data, gate):
        sl = slice(i * self.Sp, (i + 1) * self.Sp)
        used = self.zero_used if i == 0 else self.enc[i - 1][2]
        # the send buffer only feeds the packing copy, which reads the used rows: no tail zero-fill
        ops.moe_encode(data[sl], gate[sl], used, self.cf, gate_is_logits=self.gate_is_logits, zero_tail=False,
                       workspace=self.ws[i], out=self.enc[i])

    def _route(self, i, gate):
        sl = slice(i * self.Sp, (i + 1) * self.Sp)
        used = self.zero_used if i == 0 else self.enc[i - 1][2]
        ops.moe_route(gate[sl], used, self.M, self.cf, gate_is_logits=self.gate_is_logits, workspace=self.ws[i],
                      out=self.enc[i])

    def _scatter(self, i, data):
        sl = slice(i * self.Sp, (i + 1) * self.Sp)
        used = self.zero_used if i == 0 else self.enc[i - 1][2]
        ops.moe_scatter(data[sl], self.enc[i][1], used, self.enc[i][2], self.E, self.C, zero_tail=False,
                        out=self.enc[i][4])

    def _exchange(self, i):
        _, _, _, elems, disp = self.enc[i]
        ops.memcpy_sparse_to_cont_3d(disp, self.wire[i], elems, axis=0)
        ops.memcpy_cont_to_sparse_3d(self.wire[i], self.recv[i], elems, axis=0, zero_tail=True)

    def _decode(self, i):
        gates_s, indloc = self.enc[i][0], self.enc[i][1]
        ops.moe_decode(self.recv[i], gates_s, indloc, out=self.out[i * self.Sp:(i + 1) * self.Sp])

    # ---- schedules ----------------------------------------------------------------------------
    def run_serial(self, data, gate):
        """Every stage of every partition on the current stream, in pipeline order."""
        for i in range(self.P):
            self._encode(i, data, gate)
            self._exchange(i)
            self._decode(i)
        return self.out

    def run(self, data, gate):
        """Routing of all partitions on one stream, row movement (scatter, decode) on a second, exchanges on
        a third: the exchange of partition i runs beside the scatter of partition i+1, the decode of
        partition i after its exchange.  Returns the output; the caller's current stream waits for the
        pipeline before it may use it."""
        cur = torch.cuda.current_stream()
        start = torch.cuda.Event()
        start.record(cur)
        for s in (self.routing, self.compute, self.exchange):
            s.wait_event(start)
        with torch.cuda.stream(self.routing):
            for i in range(self.P):
                self._route(i, gate)
                self.routed[i].record(self.routing)
        for i in range(self.P):
            with torch.cuda.stream(self.compute):
                self.compute.wait_event(self.routed[i])
                self._scatter(i, data)
                self.encoded[i].record(self.compute)
                if i > 0:
                    self.compute.wait_event(self.received[i - 1])
                    self._decode(i - 1)
            with torch.cuda.stream(self.exchange):
                self.exchange.wait_event(self.encoded[i])
                self._exchange(i)
                self.received[i].record(self.exchange)
        with torch.cuda.stream(self.compute):
            self.compute.wait_event(self.received[self.P - 1])
            self._decode(self.P - 1)
            done = torch.cuda.Event()
            done.record(self.compute)
        cur.wait_event(done)
        return self.out

    def run_routed_once(self, data, gate):
        """The same partitions as token ranges of one routing of the whole batch: see RoutedOnceMoeLayer."""
        return self.once.run(data, gate)

    def kept_masks(self):
        """indices_locations of every partition, the input moe_merge_masks takes."""
        return [e[1] for e in self.enc]


class RoutedOnceMoeLayer:
    """The partitioned layer with the partitions taken as token ranges of ONE routing of the whole batch (the chained
    partition encodes, merged, are that routing; for top-2 in GShard's capacity order: all first choices, then all
    second choices).  Routing and the partitions' row ranges come first; then, per partition, the scatter of its
    tokens into the shared send buffer (each token row read once, also for top-2), the exchange of the rows it owns
    there (packed and unpacked at its ranges, one range per slot and expert) and the decode of its tokens from the
    shared receive buffer.  The output equals moe_decode(moe_encode(whole batch)); no buffer is per partition but
    the packed streams."""

    def __init__(self, S, M, E, n_partitions, capacity_factor=1.0, top_k=1, dtype=torch.float32, gate_is_logits=False,
                 device="cuda", streams=None):
        if S % n_partitions != 0:
            raise ValueError("the token count must divide into n_partitions")
        self.S, self.M, self.E, self.P, self.K = S, M, E, n_partitions, top_k
        self.Sp = S // n_partitions
        self.cf = float(capacity_factor)
        self.gate_is_logits = gate_is_logits
        self.C = ops.moe_capacity(S, E, self.cf * (2.0 if top_k == 2 else 1.0))
        dev = torch.device(device)
        P, K, Sp = n_partitions, top_k, self.Sp
        self.whole = (torch.empty(K * S, dtype=torch.float32, device=dev), torch.empty((2, K * S), dtype=torch.int32, device=dev),
                      torch.empty(E, dtype=torch.int32, device=dev), torch.empty(E, dtype=torch.int64, device=dev))
        with torch.cuda.device(dev):   # set up on the current stream, used on the routing stream
            self.whole_ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, K), dev)
            torch.cuda.current_stream().synchronize()
        self.ranges = (torch.empty((K * P, E), dtype=torch.int64, device=dev),
                       torch.empty((K * P, E), dtype=torch.int64, device=dev))
        self.ranges_ws = torch.empty(max(4, K * P * E * 4), dtype=torch.uint8, device=dev)
        self.send = torch.empty((E, self.C, M), dtype=dtype, device=dev)
        self.recv = torch.empty((E, self.C, M), dtype=dtype, device=dev)
        # packed streams: one per partition and slot (a partition sends at most Sp rows per slot)
        self.wire = [[torch.empty(Sp * M, dtype=dtype, device=dev) for _ in range(K)] for _ in range(P)]
        self.out = torch.empty((S, M), dtype=dtype, device=dev)
        self.no_rows = torch.empty((0, M), dtype=dtype, device=dev)
        self.routing, self.compute, self.exchange = streams or tuple(torch.cuda.Stream(device=dev) for _ in range(3))
        self.routed = torch.cuda.Event()
        self.scattered = [torch.cuda.Event() for _ in range(P)]
        self.received = [torch.cuda.Event() for _ in range(P)]

    def run(self, data, gate):
        P, K, Sp, E, C = self.P, self.K, self.Sp, self.E, self.C
        cur = torch.cuda.current_stream()
        start = torch.cuda.Event()
        start.record(cur)
        for s in (self.routing, self.compute, self.exchange):
            s.wait_event(start)
        g, il, used, _ = self.whole
        starts, counts = self.ranges
        with torch.cuda.stream(self.routing):
            ops.moe_route(gate, None, self.M, self.cf, top_k=K, gate_is_logits=self.gate_is_logits,
                          workspace=self.whole_ws, out=self.whole)
            ops.moe_partition_ranges(il, P, E, self.M, top_k=K, workspace=self.ranges_ws, out=self.ranges)
            # rows of the receive buffer no partition owns: cleared once (a scatter of no tokens is only the tail fill)
            ops.moe_scatter_tokens(self.no_rows, il, None, used, 0, E, C, top_k=K, zero_tail=True, out=self.recv)
            self.routed.record(self.routing)
        self.compute.wait_event(self.routed)
        self.exchange.wait_event(self.routed)

        def decode(i):
            ops.moe_decode_tokens(self.recv, g, il, i * Sp, Sp, top_k=K, out=self.out[i * Sp:(i + 1) * Sp])

        for i in range(P):
            with torch.cuda.stream(self.compute):
                ops.moe_scatter_tokens(data[i * Sp:(i + 1) * Sp], il, None, used, i * Sp, E, C, top_k=K, zero_tail=False,
                                       out=self.send)
                self.scattered[i].record(self.compute)
                if i > 0:
                    self.compute.wait_event(self.received[i - 1])
                    decode(i - 1)
            with torch.cuda.stream(self.exchange):
                self.exchange.wait_event(self.scattered[i])
                for j in range(K):
                    q = j * P + i
                    ops.memcpy_sparse_ranges_to_cont_3d(self.send, self.wire[i][j], counts[q], starts[q], axis=0)
                    ops.memcpy_cont_to_sparse_ranges_3d(self.wire[i][j], self.recv, counts[q], starts[q], axis=0)
                self.received[i].record(self.exchange)
        with torch.cuda.stream(self.compute):
            self.compute.wait_event(self.received[P - 1])
            decode(P - 1)
            done = torch.cuda.Event()
            done.record(self.compute)
        cur.wait_event(done)
        return self.out
