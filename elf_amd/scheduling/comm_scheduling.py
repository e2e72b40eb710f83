"""Communication ops and their ordering.

``add_comms`` appends the RECV / SEND ops each F and B needs (from the stage signatures) and one
ALL_REDUCE_PARAM_GRADS per stage; the three comm schedulers reorder the list so that matching
send / recv pairs cannot deadlock while the order of compute ops on every rank is untouched.

Behaviour follows the reference's elf/scheduling/comm_scheduling.py: DirectedGraph :13-169,
topological_sort :172-233, smart_topological_sort :236-343, pipelined_topological_sort :346-450,
schedule_to_graph :453-554, add_comms :557-598.  Dependency edges point from an op to what it
waits for; a send and its matching recv depend on each other (a 2-cycle) and are released
together.
"""

from collections import defaultdict

import numpy as np

from .scheduling import Operation, OperationType, comm_types, compute_types, get_peer, matching

__all__ = [
	"DirectedGraph", "add_comms", "schedule_to_graph", "topological_sort", "smart_topological_sort",
	"pipelined_topological_sort",
]

_T = OperationType
_RECVS = {_T.RECV_FORWARD, _T.RECV_BACKWARD}
_SENDS = {_T.SEND_FORWARD, _T.SEND_BACKWARD}


class DirectedGraph:
	"""Small directed graph over nodes 0..n-1 with O(1) edge queries (boolean matrix) and
	insertion-ordered adjacency lists."""

	def __init__(self, num_nodes):
		if num_nodes <= 0:
			raise ValueError("Number of nodes must be positive")
		self.num_nodes = num_nodes
		self.adjacency_list = defaultdict(list)
		self.reverse_adjacency_list = defaultdict(list)
		self.adjacency_matrix = np.zeros((num_nodes, num_nodes), dtype=bool)

	def _check(self, *nodes):
		if any(not (0 <= n < self.num_nodes) for n in nodes):
			raise ValueError("Node indices must be within valid range")

	def add_edge(self, source, target):
		self._check(source, target)
		if source == target:
			raise ValueError("Self-loops are not allowed")
		if not self.adjacency_matrix[source, target]:
			self.adjacency_matrix[source, target] = True
			self.adjacency_list[source].append(target)
			self.reverse_adjacency_list[target].append(source)

	def remove_edge(self, source, target):
		if self.has_edge(source, target):
			self.adjacency_matrix[source, target] = False
			self.adjacency_list[source].remove(target)
			self.reverse_adjacency_list[target].remove(source)

	def has_edge(self, source, target):
		return bool(self.adjacency_matrix[source, target])

	def has_unidirectional_edge(self, a, b):
		return self.has_edge(a, b) and not self.has_edge(b, a)

	def has_bidirectional_edge(self, a, b):
		return self.has_edge(a, b) and self.has_edge(b, a)

	def get_successors(self, node):
		return list(self.adjacency_list[node])

	def get_predecessors(self, node):
		return list(self.reverse_adjacency_list[node])

	def get_in_degree(self, node):
		return len(self.reverse_adjacency_list[node])

	def get_out_degree(self, node):
		return len(self.adjacency_list[node])

	def has_cycle(self):
		"""True if there is a cycle longer than 2 (mutual edges between two nodes do not count)."""
		state = [0] * self.num_nodes  # 0 unseen, 1 on the DFS stack, 2 finished

		def visit(node, parent):
			if state[node] == 1:
				return True
			if state[node] == 2:
				return False
			state[node] = 1
			for nxt in self.get_successors(node):
				if nxt == parent and self.has_edge(nxt, node):
					continue  # a 2-cycle with the node we came from
				if visit(nxt, node):
					return True
			state[node] = 2
			return False

		return any(state[n] == 0 and visit(n, -1) for n in range(self.num_nodes))


# --------------------------------------------------------------------------------------------
_WAITS_FOR = {
	_T.FORWARD: _T.RECV_FORWARD,
	_T.SEND_FORWARD: _T.FORWARD,
	_T.BACKWARD_INPUTS: _T.RECV_BACKWARD,
	_T.SEND_BACKWARD: _T.BACKWARD_INPUTS,
	_T.RECV_BACKWARD: _T.LOSS_BACKWARD,
}
# ops chained in list order on their rank (all-reduce and prefetch are pinned in place this way)
_CHAINED = {
	_T.FORWARD, _T.BACKWARD_INPUTS, _T.BACKWARD_PARAMS, _T.LOSS_FORWARD, _T.LOSS_BACKWARD, _T.RECOMPUTE_FORWARD,
	_T.RECOMPUTE_BACKWARD_INPUTS, _T.ALL_REDUCE_PARAM_GRADS, _T.PREFETCH_ACTIVATIONS,
}


def schedule_to_graph(schedule):
	"""Dependency graph of a schedule; node i is ``schedule[i]``, edge i -> j means i waits for j."""
	graph = DirectedGraph(len(schedule))
	by_key = {}  # (block, mb) -> [(index, op)]; ops without a micro-batch use mb -1
	for i, op in enumerate(schedule):
		by_key.setdefault((op.block_id, -1 if op.mb_id is None else op.mb_id), []).append((i, op))

	for i, op in enumerate(schedule):
		if op.op in comm_types:
			# the other end: same micro-batch on the peer block, matching type, pointing back here
			want = matching(op.op)
			for j, other in by_key.get((get_peer(op), op.mb_id), []):
				if other.op == want and get_peer(other) == op.block_id:
					graph.add_edge(i, j)
					graph.add_edge(j, i)
					break
		dep = _WAITS_FOR.get(op.op)
		if dep is not None:
			for j, other in by_key.get((op.block_id, op.mb_id), []):
				if other.op == dep:
					graph.add_edge(i, j)

	last_on_rank = {}
	for i, op in enumerate(schedule):
		if op.op in _CHAINED:
			if op.rank in last_on_rank:
				graph.add_edge(i, last_on_rank[op.rank])
			last_on_rank[op.rank] = i
	return graph


def _unmet_and_pairs(graph):
	unmet = [graph.get_out_degree(n) for n in range(graph.num_nodes)]
	pairs = {}
	for n in range(graph.num_nodes):
		for m in graph.get_predecessors(n):
			if graph.has_bidirectional_edge(n, m):
				pairs[n] = m
	return unmet, pairs


def topological_sort(schedule):
	"""Plain queue-based order; a send and its recv are emitted back to back."""
	graph = schedule_to_graph(schedule)
	unmet, pairs = _unmet_and_pairs(graph)

	def ready(n):
		if unmet[n] == 0:
			return True
		return unmet[n] == 1 and n in pairs and unmet[pairs[n]] == 1

	queue = [n for n in range(graph.num_nodes) if ready(n)]
	result = []

	def emit(n):
		result.append(schedule[n])
		for m in graph.get_predecessors(n):
			unmet[m] -= 1
			if ready(m):
				queue.append(m)
		unmet[n] = -1

	while queue:
		n = queue.pop(0)
		if unmet[n] == -1:
			continue
		emit(n)
		if n in pairs:
			emit(pairs[n])
	assert len(result) == graph.num_nodes, f"Not all nodes were visited ({len(result)}/{graph.num_nodes})"
	return result


class _Sim:
	"""State shared by the two simulation-based sorts."""

	def __init__(self, schedule):
		self.schedule = schedule
		self.graph = schedule_to_graph(schedule)
		self.unmet, self.pairs = _unmet_and_pairs(self.graph)
		# Operation hashes on (block, mb, rank, type) and compares without block_id: later equal
		# ops overwrite earlier ones here, exactly as a dict keyed by the ops themselves does
		self.node_of = {op: i for i, op in enumerate(schedule)}
		self.rank_ops = {}
		for op in schedule:
			self.rank_ops.setdefault(op.rank, []).append(op)

	def ready(self, n):
		if self.unmet[n] == 0:
			return True
		return n in self.pairs and self.unmet[n] <= 1 and self.unmet[self.pairs[n]] <= 1

	def op_ready(self, op):
		return self.ready(self.node_of[op])

	def done(self, n):
		for m in self.graph.get_predecessors(n):
			self.unmet[m] -= 1
		self.unmet[n] = -1


def smart_topological_sort(schedule):
	"""Time-stepped simulation: before each step every ready send is emitted together with its
	recv; then each rank drains its peer-less / loss / all-reduce ops and runs one compute op."""
	sim = _Sim(schedule)
	result = []

	def finish(n):
		result.append(schedule[n])
		sim.done(n)

	for n in [i for i in range(len(schedule)) if sim.ready(i)]:
		finish(n)

	while True:
		both_ends = []
		for rank, ops in sim.rank_ops.items():
			for op in [o for o in ops if sim.op_ready(o) and o.op in _SENDS]:
				n = sim.node_of[op]
				if n not in sim.pairs:
					continue
				both_ends.append(n)
				sim.rank_ops[rank].remove(op)
				peer = schedule[sim.pairs[n]]
				sim.rank_ops[peer.rank].remove(peer)
				both_ends.append(sim.pairs[n])
		for n in both_ends:
			finish(n)

		for rank, ops in sim.rank_ops.items():
			def loose():
				return [o for o in ops if sim.op_ready(o) and o.op not in compute_types and sim.node_of[o] not in sim.pairs]

			batch = loose()
			while batch:
				for op in batch:
					finish(sim.node_of[op])
					sim.rank_ops[rank].remove(op)
				batch = loose()
			for op in [o for o in ops if sim.op_ready(o)]:
				if op.op in compute_types:
					finish(sim.node_of[op])
					sim.rank_ops[rank].remove(op)
					break
		if len(result) == len(schedule):
			return result


def pipelined_topological_sort(schedule):
	"""Round-based simulation that pipelines recv -> compute -> send: in every round each rank
	first drains its ready non-compute, non-transfer ops, then starts at most one ready recv,
	runs at most one ready compute op and starts at most one ready send; transfers started in a
	round complete at its end."""
	sim = _Sim(schedule)
	result = []

	while True:
		in_flight = []
		for rank, ops in sim.rank_ops.items():
			batch = [o for o in ops if sim.op_ready(o) and o.op not in compute_types and o.op not in comm_types]
			while batch:
				for op in batch:
					result.append(op)
					sim.done(sim.node_of[op])
					sim.rank_ops[rank].remove(op)
				# from the second sweep on, peer-less transfers (the pipeline's own input / output)
				# count as drainable too
				batch = [o for o in ops if sim.op_ready(o) and o.op not in compute_types and sim.node_of[o] not in sim.pairs]

			recv = next((o for o in ops if o.op in _RECVS and sim.op_ready(o)), None)
			if recv is not None:
				result.append(recv)
				in_flight.append(sim.node_of[recv])
				sim.rank_ops[rank].remove(recv)

			comp = next((o for o in ops if o.op in compute_types and sim.op_ready(o)), None)
			if comp is not None:
				sim.rank_ops[rank].remove(comp)
				result.append(comp)
				sim.done(sim.node_of[comp])  # immediately, so that its send can start this round

			send = next((o for o in ops if o.op in _SENDS and sim.op_ready(o)), None)
			if send is not None:
				result.append(send)
				in_flight.append(sim.node_of[send])
				sim.rank_ops[rank].remove(send)

		for n in in_flight:
			sim.done(n)
		if len(result) == len(schedule):
			break

	order = [sim.node_of[op] for op in result]
	for a in range(len(order)):
		for b in range(a + 1, len(order)):
			assert not sim.graph.has_unidirectional_edge(order[a], order[b]), (
				"Backward edge found in the toposort! The schedule with reordered communications can hang."
				+ f" {order[a]} -> {order[b]}"
			)
	return result


# --------------------------------------------------------------------------------------------
def add_comms(schedule, signatures):
	"""Append, for every F (B) whose block does not have them yet, one RECV_FORWARD per source
	block (descending) and one SEND_FORWARD per target block (ascending) - for B the roles of
	sources and targets swap - then one ALL_REDUCE_PARAM_GRADS per (block, rank).  The list is
	extended in place and returned."""
	plan = {
		_T.FORWARD: (_T.RECV_FORWARD, _T.SEND_FORWARD),
		_T.BACKWARD_INPUTS: (_T.RECV_BACKWARD, _T.SEND_BACKWARD),
	}

	def present(kind, block, mb):
		return any(o.op == kind and o.block_id == block and o.mb_id == mb for o in schedule)

	for op in schedule:  # the list grows while we walk it; the appended ops are transfers and are skipped
		if op.op not in plan:
			continue
		recv_kind, send_kind = plan[op.op]
		sig = signatures[op.block_id]
		forward = op.op == _T.FORWARD

		def upstream():
			return sorted(sig.get_all_sources(), reverse=True)

		def downstream():
			return sorted(sig.get_all_targets())

		if not present(recv_kind, op.block_id, op.mb_id):
			for src in (upstream() if forward else downstream()):
				schedule.append(Operation(op.block_id, op.mb_id, recv_kind, op.rank, src=src))
		if not present(send_kind, op.block_id, op.mb_id):
			for dst in (downstream() if forward else upstream()):
				schedule.append(Operation(op.block_id, op.mb_id, send_kind, op.rank, dst=dst))

	for block, rank in set((o.block_id, o.rank) for o in schedule):
		schedule.append(Operation(block, None, _T.ALL_REDUCE_PARAM_GRADS, rank))
	return schedule
