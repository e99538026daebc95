"""A harness that builds one mixer with a cache of its own and feeds it lanes of normed inputs (GPU tests)."""
import torch

DEV = "cuda:0"


class PartHarness:
    """Builds one mixer with a cache of its own and feeds it lanes of normed inputs."""

    def __init__(self, spec, tensors, hidden, dtype, page_size=8, capacity=512, requests=4):
        from macllm_infer_amd.cache import CacheManager
        from macllm_infer_amd.kernels import build
        from macllm_infer_amd.parts import BuildContext, part_class
        cls = part_class(spec)
        build.ensure_modules(cls.kernel_modules)
        self.build = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=4096)
        self.part = cls(spec, "p", {f"p.{name}": value for name, value in tensors.items()}, self.build)
        self.cache = CacheManager({(0, "p"): cls.cache_needs(spec)}, {}, page_size, capacity, requests, dtype, DEV)

    def run(self, lanes):
        """lanes: [(request, x [t, hidden])] -> outputs per lane."""
        from macllm_infer_amd.engine import Lane, build_step_context
        for request, x in lanes:
            if request not in self.cache.requests:
                self.cache.add_request(request)
        self.cache.reserve([(request, x.shape[0]) for request, x in lanes])
        step = build_step_context([Lane(request, [0] * x.shape[0]) for request, x in lanes], self.cache, DEV,
                                  query_tile=getattr(self.part, "query_tile", 0),
                                  chunk_sizes=tuple({getattr(self.part, "chunk_tokens", 0)} - {0}))
        x = torch.cat([x for _, x in lanes]).to(self.build.dtype).to(DEV)
        out = self.part.forward(x, step, self.cache.entry((0, "p"))).float().cpu()
        pieces, cursor = [], 0
        for request, lane_x in lanes:
            self.cache.commit(request, lane_x.shape[0])
            pieces.append(out[cursor:cursor + lane_x.shape[0]])
            cursor += lane_x.shape[0]
        return pieces
