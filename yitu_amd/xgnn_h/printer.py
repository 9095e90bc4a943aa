"""Text dump of a dataflow graph (the role of xgnn_h/printer.py): one line per
node in evaluation order, ``%id: size = op(slot: %id, ...)``."""
import sys

from . import ir


class Printer:
    def dump(self, dataflow: ir.Dataflow, file=None):
        out = file or sys.stdout
        ids = {}
        for node in ir.walk(dataflow):
            label = node.name if node.op in ("input", "graph") else str(
                sum(1 for n in ids.values() if n.isdigit()))
            ids[id(node)] = label
            op = node.op
            if "fn" in node.attrs:
                op += "." + node.fn_name()
            args = ", ".join("%s: %%%s" % (k, ids[id(v)]) for k, v in node.inputs.items())
            size = ": %s" % (node.size,) if node.size is not None else ""
            print("%%%s%s = %s(%s)" % (label, size, op, args), file=out)
