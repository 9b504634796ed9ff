"""HIP graph capture of a sequence of kernel calls (launch-bound inner loops are replayed with one host call).

The capture runs inside a memory arena of its own: eager passes first fill the arena's free lists, the captured pass then
finds every block it asks for there (the capture never reaches the driver's allocator, which is not allowed while a stream
is capturing), and afterwards nobody else is handed the addresses the graph has baked in.  A function that keeps results of
one call alive into the next (a training step that replaces its parameters) needs more than one eager pass before a pass
allocates nothing new; the passes are repeated until that is the case.  PyTorch provides the capture itself
(``torch.cuda.CUDAGraph``) and the stream.
"""
import gc

from chainer_amd._array import memory_arena, pool_stats, torch

MAX_WARM_PASSES = 4


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
    """Runs ``fn()`` eagerly until a pass gets all its memory from the arena's free lists, then once under capture; returns a
    CapturedGraph."""
    t = torch()
    arena = memory_arena()
    # both passes run on one side stream: the pool keeps the blocks of different streams apart
    stream = t.cuda.Stream()
    stream.wait_stream(t.cuda.current_stream())
    try:
        with arena:
            for _ in range(MAX_WARM_PASSES):
                gc.collect()  # arrays held only by garbage cycles would otherwise be freed at some later, arbitrary moment
                before = pool_stats()['device_allocations']
                with t.cuda.stream(stream):
                    out = fn()
                stream.synchronize()
                del out
                if pool_stats()['device_allocations'] == before:
                    break
            else:
                raise RuntimeError('capture: fn() still took new memory from the driver in each of its %d warm passes (it allocates more '
                                   'from pass to pass, e.g. by keeping its results alive); a pass that allocates cannot be captured'
                                   % MAX_WARM_PASSES)
            gc.collect()
            graph = t.cuda.CUDAGraph()
            with t.cuda.graph(graph, stream=stream):
                out = fn()
    except BaseException:
        arena.release()  # its cached blocks join the general pool again
        raise
    return CapturedGraph(graph, out, arena)
