"""Directed graph used for the op DAG and the device topology.

Interface and ordering rules follow the reference's ``pccl/lang/utils/graph.py``:
``add_node`` hands out dense ids in insertion order and ignores any id the caller had in mind
(graph.py:23-27), ``add_edge`` rejects unknown ids with ``ValueError("Invalid node IDs")``
(graph.py:29-36), and ``topological_sort`` is the reverse post-order of a depth-first search
that starts from nodes in id order and follows successors in edge-insertion order
(graph.py:94-112).  The traversals here are iterative, so DAG depth is not bounded by the
interpreter's recursion limit.
"""


class DirectedGraph:
    def __init__(self):
        self._data = []   # node id -> payload
        self._succ = []   # node id -> successor ids, edge insertion order
        self._pred = []
        self._edges = []  # (src, dst, data)

    # -- construction ---------------------------------------------------------------------
    def add_node(self, data=None):
        self._data.append(data)
        self._succ.append([])
        self._pred.append([])
        return len(self._data) - 1

    def add_edge(self, src_id, dst_id, data=None):
        n = len(self._data)
        if not (isinstance(src_id, int) and isinstance(dst_id, int) and 0 <= src_id < n and 0 <= dst_id < n):
            raise ValueError("Invalid node IDs")
        self._edges.append((src_id, dst_id, data))
        self._succ[src_id].append(dst_id)
        self._pred[dst_id].append(src_id)

    def remove_edge(self, src_id, dst_id):
        for i, (s, d, _) in enumerate(self._edges):
            if s == src_id and d == dst_id:
                del self._edges[i]
                self._succ[s].remove(d)
                self._pred[d].remove(s)
                return

    # -- queries --------------------------------------------------------------------------
    @property
    def nodes(self):
        return {i: self._data[i] for i in range(len(self._data))}

    def num_nodes(self):
        return len(self._data)

    def get_node(self, node_id):
        return self._data[node_id] if 0 <= node_id < len(self._data) else None

    def get_edges(self):
        return list(self._edges)

    def get_predecessors(self, node_id):
        return list(self._pred[node_id]) if 0 <= node_id < len(self._data) else []

    def get_successors(self, node_id):
        return list(self._succ[node_id]) if 0 <= node_id < len(self._data) else []

    # -- traversals -----------------------------------------------------------------------
    def _post_order(self):
        """Returns (post_order, acyclic)."""
        n = len(self._data)
        state = [0] * n  # 0 unvisited, 1 on the stack, 2 finished
        post = []
        for root in range(n):
            if state[root]:
                continue
            stack = [(root, 0)]
            state[root] = 1
            while stack:
                v, i = stack[-1]
                if i < len(self._succ[v]):
                    stack[-1] = (v, i + 1)
                    w = self._succ[v][i]
                    if state[w] == 1:
                        return post, False
                    if state[w] == 0:
                        state[w] = 1
                        stack.append((w, 0))
                else:
                    state[v] = 2
                    post.append(v)
                    stack.pop()
        return post, True

    def is_acyclic(self):
        return self._post_order()[1]

    def topological_sort(self):
        post, ok = self._post_order()
        if not ok:
            raise ValueError("Graph contains cycles")
        return post[::-1]

    def get_connected_components(self):
        n = len(self._data)
        seen = [False] * n
        comps = []
        for root in range(n):
            if seen[root]:
                continue
            comp, stack = [], [root]
            seen[root] = True
            while stack:
                v = stack.pop()
                comp.append(v)
                # successors first, then predecessors, like the reference's dfs (graph.py:118-126)
                for w in reversed(self._succ[v] + self._pred[v]):
                    if not seen[w]:
                        seen[w] = True
                        stack.append(w)
            comps.append(comp)
        return comps
