"""Comparison switches of the Python host side.

Every default is the fast path; a switch exists so that a run can be compared with the path it replaced
(and so that tests can hold both to the same results).  The environment is read ONCE, when this module is
imported, into one object; the operators read that object when they are called, so a test may flip a field
for the duration of a call.  The library's own switches (tile shapes, block orders) are read the same way
inside the library when it is loaded (``csrc/mts_tuning.h``).

    MTS_NO_OVERLAP=1          every kernel of the backward pass on the caller's stream (no side streams)
    MTS_NO_JOINT_BWD=1        dW2, dW1 and dX as launches of their own even where one launch could hold them
    MTS_NO_TAIL_IN_JOINT=1    the router's backward of the layer node in launches of its own
    MTS_NO_COMBINE_IN_TAIL=1  the dX combine behind the joint launch in a launch of its own
    MTS_NO_JOINT_FWD=1        gate/up and down as two launches even where one launch could hold them
    MTS_NO_JOINT_SCHEDULE=1   no table for the joint launch: its blocks are dealt to the XCDs without regard to routing
    MTS_WEIGHTED_POST=0       the forward pass writes the unweighted activation and dO*W2 writes s * a again
    MTS_NO_ROUTER_CAST=1      router_postprocess leaves the cast of the routing weights to the caller
    MTS_NO_LAYER_NODE=1       the backend does not offer the layer as one autograd node (the block composes it)
"""

import os
from dataclasses import dataclass


def _off(name: str) -> bool:
    """A switch is set when its value parses to a non-zero integer ("0" and the empty string leave it alone)."""
    try:
        return int(os.environ.get(name, "0") or "0") != 0
    except ValueError:
        return False


@dataclass
class Switches:
    overlap: bool
    joint_bwd: bool
    joint_fwd: bool
    tail_in_joint: bool
    combine_in_tail: bool
    joint_schedule: bool
    weighted_post: bool
    router_cast: bool
    layer_node: bool


SWITCHES = Switches(
    overlap=not _off("MTS_NO_OVERLAP"),
    joint_bwd=not _off("MTS_NO_JOINT_BWD"),
    joint_fwd=not _off("MTS_NO_JOINT_FWD"),
    tail_in_joint=not _off("MTS_NO_TAIL_IN_JOINT"),
    combine_in_tail=not _off("MTS_NO_COMBINE_IN_TAIL"),
    joint_schedule=not _off("MTS_NO_JOINT_SCHEDULE"),
    weighted_post=os.environ.get("MTS_WEIGHTED_POST", "1") != "0",
    router_cast=not _off("MTS_NO_ROUTER_CAST"),
    layer_node=not _off("MTS_NO_LAYER_NODE"),
)
