"""HIP graph capture of a sequence of kernel calls (launch-bound inner loops are replayed with one host call).

The capture runs inside a memory arena of its own: an eager pass first fills the arena's free lists, the captured pass then
finds every block it asks for there (the capture never reaches the driver's allocator, which is not allowed while a stream
is capturing), and afterwards nobody else is handed the addresses the graph has baked in.  PyTorch provides the capture
itself (``torch.cuda.CUDAGraph``) and the stream.
"""
from chainer_amd._array import memory_arena, torch


class CapturedGraph(object):
    def __init__(self, graph, result, arena):
        self.graph = graph
        self.result = result  # what fn() returned inside the capture: rewritten by every replay
        self.arena = arena

    def replay(self):
        self.graph.replay()

    def release(self):
        """Drops the graph; its blocks return to the general pool once the arrays that refer to them are gone."""
        self.graph = None
        self.result = None
        self.arena.release()


def capture(fn):
    """Runs ``fn()`` once eagerly and once under capture; returns a CapturedGraph."""
    t = torch()
    arena = memory_arena()
    # both passes run on one side stream: the pool keeps the blocks of different streams apart
    stream = t.cuda.Stream()
    stream.wait_stream(t.cuda.current_stream())
    with arena:
        with t.cuda.stream(stream):
            out = fn()
        stream.synchronize()
        del out
        graph = t.cuda.CUDAGraph()
        with t.cuda.graph(graph, stream=stream):
            out = fn()
    return CapturedGraph(graph, out, arena)
