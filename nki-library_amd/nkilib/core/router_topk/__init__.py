from .router_topk import route_for_moe, router_topk

__all__ = ["router_topk", "route_for_moe"]
