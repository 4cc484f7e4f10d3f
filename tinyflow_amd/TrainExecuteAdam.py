"""Adam training-step executor.

Counterpart of the reference ``pycode/tinyflow/TrainExecuteAdam.py``: the step
graph of ``TrainExecute.TrainExecutor`` with one ``adam_op`` per variable in place
of the SGD node.  Every variable gets two moment variables, ``<name>m`` and
``<name>v``, that start at zero (reference TrainExecuteAdam.py:80-86) and live on
the device next to the parameter.  The bias-correction powers start at b1 and b2
and are multiplied by b1 and b2 after every step (reference :16-21, :196-198), so
step t (counted from 1) corrects with 1 - b1^t and 1 - b2^t.
"""
import numpy as np

from . import autodiff as ad
from . import ndarray
from . import TrainExecute as _sgd


class TrainExecutor(_sgd.TrainExecutor):
    """Runs forward + backward + Adam update for one loss node."""

    def __init__(self, targetloss, learning_rate=0.001, ctx=ndarray.gpu(0), fuse_bn_relu=False):
        self.b1 = 0.9
        self.b2 = 0.999
        self.e = 0.00000001
        self.b1t = [0.9]
        self.b2t = [0.999]
        self.mv = []
        self.Variable_node_to_mv = {}
        _sgd.TrainExecutor.__init__(self, targetloss, learning_rate, ctx, fuse_bn_relu)

    def _update_nodes(self):
        nodes, self.mv, self.Variable_node_to_mv = getcomputelist(
            self.Variable_node_list, self.Variable_node_grad_list, self.b1, self.b2, self.b1t, self.b2t, self.e,
            self.learning_rate)
        return nodes

    def init_Variable(self, feed_dict):
        """Initial values (numpy) of the trainable variables; the moments start at zero."""
        values = dict(feed_dict)
        for node in self.Variable_node_list:
            m, v = self.Variable_node_to_mv[node]
            values[m] = np.zeros(np.shape(feed_dict[node]), dtype=np.float32)
            values[v] = np.zeros(np.shape(feed_dict[node]), dtype=np.float32)
        self.Variable_node_np_value = values

    def run(self, feed_dict, Accuracy_node=None, convert_to_numpy_ret_vals=False):
        """One step.  Returns [loss, variables in network order (, accuracy node)]."""
        result = _sgd.TrainExecutor.run(self, feed_dict, Accuracy_node, convert_to_numpy_ret_vals)
        self.b1t[0] = self.b1t[0] * self.b1
        self.b2t[0] = self.b2t[0] * self.b2
        return result

    def moments_of(self, variable):
        """Device arrays (m, v) of a trainable variable."""
        m, v = self.Variable_node_to_mv[variable]
        return self.node_to_arr_map[m], self.node_to_arr_map[v]


def getcomputelist(Variable_node_list, Variable_node_grad_list, b1, b2, b1t, b2t, e, learning_rate):
    """One in-place Adam node and two moment variables per variable
    (reference TrainExecuteAdam.py:347-362)."""
    computelist, mv, var_to_mv = [], [], {}
    for var, grad in zip(Variable_node_list, Variable_node_grad_list):
        m = ad.Variable(var.name + "m")
        v = ad.Variable(var.name + "v")
        mv += [m, v]
        var_to_mv[var] = (m, v)
        node = ad.adam_op(var, m, v, grad, b1, b2, b1t, b2t, e, learning_rate)
        node.issgd = 1
        computelist.append(node)
    return computelist, mv, var_to_mv


# an update node moves behind the last reader of its parameter exactly as for SGD
# (reference TrainExecuteAdam.py:367-388)
swapadam = _sgd.swapsgd
