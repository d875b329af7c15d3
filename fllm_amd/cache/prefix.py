"""Index of prompt prefixes whose keys and values are in the cache: full pages whose tokens, and all tokens before
them, were computed once are kept after their request has ended, and a later request that begins with the same
tokens takes them over instead of computing them again (rust/engine/src/mem/prefix_cache.rs:91-640 is the
reference's, with hashes of the tokens as keys; this one is a tree keyed by the tokens of each page themselves, so two
prefixes are the same only if their tokens are).

A node stands for one page position of one prefix: the page of every cache group that holds these tokens.  The cache
manager owns the references (one of the index to each page of a node) and the order in which unused nodes are given up.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple


class PrefixNode:
    __slots__ = ("parent", "key", "pages", "children", "holders", "state")

    def __init__(self, parent: Optional["PrefixNode"], key: Tuple[int, ...], pages: Tuple[int, ...]):
        self.parent = parent
        self.key = key                   # the tokens of this page
        self.pages = pages               # one page a cache group
        self.children: Dict[Tuple[int, ...], "PrefixNode"] = {}
        self.holders = 0                 # live requests whose block tables name these pages
        self.state = None                # for models with per-request state: a copy of it as it was behind this page


class PrefixIndex:
    def __init__(self, page_size: int):
        self.page_size = page_size
        self.root = PrefixNode(None, (), ())
        self.size = 0

    def match(self, tokens: Sequence[int], max_pages: int) -> List[PrefixNode]:
        """The nodes of the longest known prefix of `tokens`, page by page, at most `max_pages` of them."""
        found: List[PrefixNode] = []
        node = self.root
        for i in range(max_pages):
            child = node.children.get(tuple(tokens[i * self.page_size:(i + 1) * self.page_size]))
            if child is None:
                break
            found.append(child)
            node = child
        return found

    def child(self, parent: Optional[PrefixNode], key: Tuple[int, ...]) -> Optional[PrefixNode]:
        return (parent or self.root).children.get(key)

    def insert(self, parent: Optional[PrefixNode], key: Tuple[int, ...], pages: Tuple[int, ...]) -> PrefixNode:
        parent = parent or self.root
        if key in parent.children:
            raise ValueError("this prefix is known already")
        node = PrefixNode(parent, key, pages)
        parent.children[key] = node
        self.size += 1
        return node

    def remove(self, node: PrefixNode) -> None:
        if node.children:
            raise ValueError("a prefix is given up from its end")
        del node.parent.children[node.key]
        self.size -= 1

    def nodes(self) -> List[PrefixNode]:
        out: List[PrefixNode] = []
        stack = list(self.root.children.values())
        while stack:
            node = stack.pop()
            out.append(node)
            stack.extend(node.children.values())
        return out
