"""SGD training-step executor.

Counterpart of the reference ``pycode/tinyflow/TrainExecute.py``: given a loss
node it collects the trainable variables, differentiates, appends one ``sgd_op``
per variable, orders everything topologically and moves each update behind the
last reader of its parameter (``swapsgd``).  The first ``run`` infers shapes
(which creates the C-side descriptors) and allocates one device array per node;
later runs copy the feeds in and recompute every node in place.

A step only enqueues work: nothing waits for the GPU except the read-back of a
(1,)-shaped operand inside Add/Mul (the upstream-gradient scalar) and whatever
the caller reads afterwards with ``asnumpy``.
"""
import numpy as np

from . import autodiff as ad
from . import gpu_op, ndarray


class TrainExecutor(object):
    """Runs forward + backward + SGD update for one loss node."""

    def __init__(self, targetloss, learning_rate, ctx=ndarray.gpu(0), fuse_bn_relu=False, fused_update=True):
        """``fuse_bn_relu`` (no counterpart in the reference): evaluate every batch
        norm whose only reader is a ReLU together with that ReLU, forward and
        backward, through the fused entry points.  Results are bit-identical; the
        batch-norm output and the ReLU's input gradient are then never materialised
        (``value_of`` does not know them).

        ``fused_update``: apply all SGD updates of a step with one call of the
        multi-tensor entry point (``sgd_compute_o``, reference gpu_op.py:939-945) behind
        the last node of the step instead of one ``sgd_update`` per variable.  Every
        update still comes after the last reader of its parameter, which is all
        ``swapsgd`` asks for, and the arithmetic per element is the same."""
        self.fuse_bn_relu = fuse_bn_relu
        self.fused_update = fused_update
        self._fused_sgd = None
        self.fused_pairs = 0
        self.targetloss = targetloss
        self.learning_rate = learning_rate
        self.Variable_node_list = ad.get_Variable_node_list(targetloss)
        self.Variable_node_list.reverse()
        self.Variable_node_grad_list = ad.gradients(targetloss, self.Variable_node_list)
        self.eval_node_list = self._update_nodes()
        self.ctx = ctx
        self.topo_order = swapsgd(ad.find_topo_sort(self.eval_node_list))
        self.node_to_shape_map = None
        self.node_to_arr_map = {}
        self.Variable_node_np_value = None
        self.cudaStream = gpu_op.create_cudaStream()
        self.cudnnHandle = gpu_op.create_cudnnHandle(self.cudaStream)
        self.cublasHandle = gpu_op.create_cublasHandle(self.cudaStream)
        self.isfirstrun = 0
        self._plan = None

    def _update_nodes(self):
        """One in-place update node per variable, in ``Variable_node_list`` order."""
        return getcomputelist(self.Variable_node_list, self.Variable_node_grad_list, self.learning_rate)

    def infer_shape(self, feed_shapes):
        """Shapes of every node from the shapes of the fed nodes."""
        self.node_to_shape_map = dict(feed_shapes)
        for node in self.topo_order:
            if node in self.node_to_shape_map:
                continue
            input_shapes = [self.node_to_shape_map[i] for i in node.inputs]
            assert None not in input_shapes
            self.node_to_shape_map[node] = tuple(node.op.infer_shape(node, input_shapes, self.cudnnHandle))

    def init_Variable(self, feed_dict):
        """Initial values (numpy) of the trainable variables, used by the first run."""
        self.Variable_node_np_value = feed_dict

    def _alloc(self, shape):
        arr = ndarray.empty(shape, ctx=self.ctx)
        if isinstance(arr, int):
            raise MemoryError("device out of memory: %d more bytes wanted" % arr)
        return arr

    def _first_run(self, feed_dict):
        feed_dict = dict(feed_dict)
        feed_dict.update(self.Variable_node_np_value or {})
        self.infer_shape({node: np.shape(value) for node, value in feed_dict.items()})
        plan = []
        fused = {}
        fused_sgd = []   # (parameter array, gradient array, learning rate) of the updates applied in one call
        if self.fuse_bn_relu:
            fused.update(find_bn_relu_pairs(self.topo_order, {self.targetloss}))
            fused.update(find_add_relu_pairs(self.topo_order, {self.targetloss}, self.node_to_shape_map))
        self.fused_pairs = sum(1 for v in fused.values() if v[0] in ("forward", "add_relu"))
        unread_zeros = _zeros_only_added(self.topo_order, self.node_to_shape_map,
                                         set(self.eval_node_list) | {self.targetloss})
        for role in fused.values():   # a fused call reads its sources as arrays
            if len(role) == 3:
                unread_zeros -= set(role[2])
        for node in self.topo_order:
            if node in unread_zeros:
                continue   # every reader adds it as the constant 0.0: never materialised
            role = fused.get(node)
            if role is not None and role[0] == "skip":
                continue   # its value is folded into the fused call of its reader
            if role is not None:
                kind, bn, sources = role
                inputs = [self.node_to_arr_map[i] for i in sources]
                node_val = self._alloc(self.node_to_shape_map[node])
                self.node_to_arr_map[node] = node_val
                plan.append((_fused_compute(kind, bn), node, inputs, node_val))
                continue
            if node in feed_dict:
                arr = ndarray.array(feed_dict[node], ctx=self.ctx)
                if isinstance(arr, int):
                    raise MemoryError("device out of memory: %d more bytes wanted" % arr)
                self.node_to_arr_map[node] = arr
                continue
            assert node.isw not in (1, 2), "no value fed for %s" % node.name
            input_vals = [self.node_to_arr_map.get(i) if i in unread_zeros else self.node_to_arr_map[i]
                          for i in node.inputs]
            if node.issgd and self.fused_update and isinstance(node.op, ad.SgdOp):
                fused_sgd.append((input_vals[0], input_vals[1], node.learning_rate))
                continue
            if node.issgd:
                node_val = None  # updates its parameter in place
            else:
                node_val = self._alloc(self.node_to_shape_map[node])
                self.node_to_arr_map[node] = node_val
            plan.append((_known_scalar_compute(node, self.node_to_shape_map)
                         or _known_zeros_compute(node, self.node_to_shape_map) or node.op.compute, node, input_vals,
                         node_val))
        self._plan = plan
        if self._fused_sgd is not None:
            self._fused_sgd.close()
            self._fused_sgd = None
        if fused_sgd:
            self._fused_sgd = _FusedSgd(fused_sgd)
        self.isfirstrun = 1

    def run(self, feed_dict, Accuracy_node=None, convert_to_numpy_ret_vals=False):
        """One step.  Returns [loss, variables in network order (, accuracy node)]."""
        if self.isfirstrun == 0:
            self._first_run(feed_dict)
        else:
            for node, value in feed_dict.items():
                if node.isw == 1:
                    continue  # variables live on the device; only data is re-fed
                self.node_to_arr_map[node]._sync_copyfrom(value)
        handles = (self.cudnnHandle, self.cublasHandle, self.cudaStream)
        for compute, node, input_vals, node_val in self._plan:
            wanted = compute(node, input_vals, node_val, *handles)
            if wanted:
                raise MemoryError("%s: %d bytes of device scratch could not be allocated" % (node.name, wanted))
        if self._fused_sgd is not None:
            self._fused_sgd.apply()
        result = [self.node_to_arr_map[self.targetloss]]
        result += [self.node_to_arr_map[v] for v in reversed(self.Variable_node_list)]
        if Accuracy_node is not None:
            result.append(self.node_to_arr_map[Accuracy_node])
        if convert_to_numpy_ret_vals:
            return [r.asnumpy() for r in result]
        return result

    def value_of(self, node):
        """Device array currently holding ``node`` (any node of the step graph)."""
        return self.node_to_arr_map[node]

    def close(self):
        """Gives the stream and the two handles back to the library (waits for the
        stream first).  The library orders copies and storage reuse against every
        stream that has run kernels, so an executor that is done should not leave
        its stream registered; the fused update's device tables go back to the pool.
        Arrays already returned stay valid."""
        if self.cudaStream is None:
            return
        stream, self.cudaStream = self.cudaStream, None
        self._plan = None
        if self._fused_sgd is not None:
            self._fused_sgd.close()
            self._fused_sgd = None
        gpu_op.destroy_cudnnHandle(self.cudnnHandle)
        gpu_op.destroy_cublasHandle(self.cublasHandle)
        gpu_op.destroy_cudaStream(stream)

    def __del__(self):
        try:
            self.close()
        except Exception:   # interpreter shutdown: the library may already be gone
            pass


class _FusedSgd(object):
    """All SGD updates of a step as one launch: the pointer tables and the index ->
    (tensor, offset) tables of ``sgd_compute_o`` (reference gpu_op.py:887-945), built
    once for the step's parameter and gradient arrays, which keep their storage from
    step to step.  The call has no stream argument: it runs on the default stream,
    which is ordered behind the executor's stream and in front of its next launch."""

    def __init__(self, updates):
        rates = set(lr for _, _, lr in updates)
        assert len(rates) == 1, "one learning rate per step"
        self.learning_rate = rates.pop()
        self.arrays = [(w, g) for w, g, _ in updates]   # keeps the storage alive
        sizes = [int(np.prod(w.shape)) for w, _ in self.arrays]
        for (w, g), n in zip(self.arrays, sizes):
            assert int(np.prod(g.shape)) == n, "gradient and parameter sizes differ"
        assert sum(sizes) < 2 ** 31
        # whole tensors end to end: the tables are built from the sizes, not from
        # per-parameter (tensor, offset) arrays
        self.tables, self.count = gpu_op.get_tensor_runs_cuda_pointer(sizes)
        self.pointers = gpu_op.get_n2_cuda_pointer([w.handle.contents.data for w, _ in self.arrays],
                                                   [g.handle.contents.data for _, g in self.arrays], len(sizes))

    def apply(self):
        gpu_op.sgd_compute_o(self.pointers, self.tables, self.count, self.learning_rate)

    def close(self):
        """Gives the device tables back (waits for the last update that reads them)."""
        if self.tables is not None:
            gpu_op.free_index_cuda_pointer(self.tables)
            gpu_op.free_n_cuda_pointer(self.pointers, 2)
            self.tables = self.pointers = None
            self.arrays = []


def find_bn_relu_pairs(topo_order, outputs):
    """Batch norms that can be evaluated together with the ReLU that follows them.

    A per-activation batch-norm node B qualifies when its only readers are a ReLU
    activation R and that activation's backward node A (which reads B as the ReLU
    input), and A's only reader is B's own backward node D.  Returns a dict:
    B and A -> ("skip",); R -> ("forward", B, [x]); D -> ("backward", B, [x, dR])."""
    readers = {}
    for n in topo_order:
        for inp in n.inputs:
            readers.setdefault(inp, []).append(n)
    roles = {}
    for r in topo_order:
        if not (isinstance(r.op, ad.ActivationForwardOp) and r.activationMode == "relu"):
            continue
        b = r.inputs[0]
        if not isinstance(b.op, ad.BNForwardOp) or b.batchNormMode != "pre_activation" or b in outputs:
            continue
        others = [n for n in readers.get(b, []) if n is not r]
        if len(others) != 1:
            continue
        a = others[0]
        if not (isinstance(a.op, ad.ActivationBackwardOp) and a.inputs[0] is b and a.inputs[2] is r) or a in outputs:
            continue
        a_readers = readers.get(a, [])
        if len(a_readers) != 1:
            continue
        d = a_readers[0]
        if not (isinstance(d.op, ad.BNBackwardOp) and d.inputs[1] is a and d.inputs[0] is b.inputs[0]
                and d.Save_p is b.Save_p):
            continue
        roles[b] = ("skip",)
        roles[a] = ("skip",)
        roles[r] = ("forward", b, [b.inputs[0]])
        roles[d] = ("backward", b, [b.inputs[0], a.inputs[1]])
    return roles


def find_add_relu_pairs(topo_order, outputs, shapes):
    """Elementwise sums that can be evaluated together with the ReLU that follows them
    (the join of a residual block).  A sum S of two equally shaped values qualifies
    when its only readers are a ReLU activation R and R's backward node A, which
    reads S only to rebuild the mask S > 0 -- and R > 0 is the same mask.  Returns
    S -> ("skip",); R -> ("add_relu", S, [a, b]); A -> ("mask_from_output", S, [R, dR, R])."""
    readers = {}
    for n in topo_order:
        for inp in n.inputs:
            readers.setdefault(inp, []).append(n)
    roles = {}
    for r in topo_order:
        if not (isinstance(r.op, ad.ActivationForwardOp) and r.activationMode == "relu"):
            continue
        s = r.inputs[0]
        if not isinstance(s.op, ad.AddOp) or s in outputs or len(s.inputs) != 2:
            continue
        if not (shapes[s.inputs[0]] == shapes[s.inputs[1]] == shapes[s]):
            continue   # a (1,)-shaped operand is applied as a constant, not added elementwise
        others = [n for n in readers.get(s, []) if n is not r]
        if len(others) != 1:
            continue
        a = others[0]
        if not (isinstance(a.op, ad.ActivationBackwardOp) and a.inputs[0] is s and a.inputs[2] is r):
            continue
        roles[s] = ("skip",)
        roles[r] = ("add_relu", s, list(s.inputs))
        roles[a] = ("mask_from_output", s, [r, a.inputs[1], r])
    return roles


def _known_scalar_compute(node, shapes):
    """Plan entry for an Add / Mul node one of whose operands is a (1,)-shaped
    ``oneslike`` / ``zeroslike`` value, or None.  The op itself reads a (1,) operand
    back to the host every step and applies it as a constant (reference
    autodiff.py:302-348, 376-413), which makes the host wait for the whole forward pass
    at the upstream-gradient scalar of the loss; the value of such a producer is 1.0 or
    0.0 whatever its input holds, so the constant is known without reading it."""
    if not isinstance(node.op, (ad.AddOp, ad.MulOp)) or len(node.inputs) != 2:
        return None
    a, b = node.inputs
    if shapes[a] == shapes[b]:
        return None
    which = 1 if shapes[b] == (1,) else 0 if shapes[a] == (1,) else None
    if which is None:
        return None
    producer = node.inputs[which]
    if isinstance(producer.op, ad.OnesLikeOp):
        constant = 1.0
    elif isinstance(producer.op, ad.ZerosLikeOp):
        constant = 0.0
    else:
        return None
    by_const = (gpu_op.matrix_elementwise_add_by_const if isinstance(node.op, ad.AddOp)
                else gpu_op.matrix_elementwise_multiply_by_const)

    def compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream):
        by_const(input_vals[1 - which], constant, output_val, cudaStream)
        return 0
    return compute


def _added_zeros_operand(node, shapes):
    """Index of the operand of an Add node that is a ``zeroslike`` of the other
    operand's shape, or None."""
    if not isinstance(node.op, ad.AddOp) or len(node.inputs) != 2:
        return None
    for which in (0, 1):
        z, other = node.inputs[which], node.inputs[1 - which]
        if isinstance(z.op, ad.ZerosLikeOp) and shapes[z] == shapes[other] and not isinstance(other.op, ad.ZerosLikeOp):
            return which
    return None


def _known_zeros_compute(node, shapes):
    """Plan entry for ``x + zeroslike(.)`` of equal shapes, or None.  The reference's
    broadcast gradient hands a zeros tensor to its second input (autodiff.py, the
    ``broadcastto`` gradient), which the accumulation of adjoints then adds to the real
    gradient: a fill and a two-operand add per bias.  Adding the constant 0.0 gives the
    same bits (x + 0.0 is the same IEEE sum) with one read less and no fill."""
    which = _added_zeros_operand(node, shapes)
    if which is None:
        return None

    def compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream):
        gpu_op.matrix_elementwise_add_by_const(input_vals[1 - which], 0.0, output_val, cudaStream)
        return 0
    return compute


def _zeros_only_added(topo_order, shapes, outputs):
    """``zeroslike`` nodes all of whose readers are such additions (and that nobody
    asks for): their value is never needed as an array."""
    readers = {}
    for n in topo_order:
        for inp in n.inputs:
            readers.setdefault(inp, []).append(n)
    unread = set()
    for z in topo_order:
        if not isinstance(z.op, ad.ZerosLikeOp) or z in outputs or not readers.get(z):
            continue
        if all((_added_zeros_operand(r, shapes) is not None and r.inputs[_added_zeros_operand(r, shapes)] is z)
               for r in readers[z]):
            unread.add(z)
    return unread


def _fused_compute(kind, bn):
    """Plan entry (same signature as ``Op.compute``) for a fused node: batch norm
    ``bn`` with its ReLU (forward / backward), a sum with its ReLU, or a ReLU backward
    that takes its mask from the ReLU output."""
    if kind == "add_relu":
        def compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream):
            assert input_vals[0].shape == input_vals[1].shape == output_val.shape
            gpu_op.matrix_elementwise_add_relu(input_vals[0], input_vals[1], output_val, cudaStream)
            return 0
        return compute
    if kind == "mask_from_output":
        def compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream):
            return node.op.compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream)
        return compute
    if kind == "forward":
        def compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream):
            wanted = gpu_op.bn_relu_forward(input_vals[0], output_val, bn.batchNormMode, bn.n, bn.Save_p[0],
                                            bn.Save_p[1], bn.cudnnlist[0], cudnnHandle, cudaStream)
            bn.n += 1
            return wanted
    else:
        def compute(node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream):
            return gpu_op.bn_relu_backward(input_vals[0], input_vals[1], output_val, bn.batchNormMode, bn.Save_p[0],
                                           bn.Save_p[1], bn.cudnnlist[0], cudnnHandle, cudaStream)
    return compute


def getcomputelist(Variable_node_list, Variable_node_grad_list, learning_rate):
    """One in-place SGD node per variable (reference TrainExecute.py:315-324)."""
    computelist = []
    for var, grad in zip(Variable_node_list, Variable_node_grad_list):
        node = ad.sgd_op(var, grad, learning_rate)
        node.issgd = 1
        computelist.append(node)
    return computelist


def swapsgd(topoorder):
    """Move every update node to just behind the last non-update node that reads
    its parameter, so that e.g. the grad-data convolution of a layer still sees
    the weights the forward pass used (reference TrainExecute.py:329-349)."""
    topoorder = list(topoorder)
    i = 0
    while i < len(topoorder):
        node = topoorder[i]
        if node.issgd == 1 and node.isw == 0:
            node.isw = 3
            param = node.inputs[0]
            j = len(topoorder) - 1
            while j > i:
                other = topoorder[j]
                if other.issgd != 1 and param in other.inputs:
                    break
                j -= 1
            if j > i:
                topoorder.pop(i)
                topoorder.insert(j, node)
                continue  # position i now holds the next node
        i += 1
    return topoorder
