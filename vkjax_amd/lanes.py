'''Which launches of a program may share the GPU with the ones before them.

The reference records one dispatch per equation into a single in-order sequence
(vkjax/kompute_jaxpr_interpreter.py:55-60). Here a recorded sequence has two lanes (two HIP streams of the
same priority, include/vkjax_hip.h: vkj_seq_set_launch_lane): launches keep their program order within a
lane, and a lane waits for the other one only where data say so. This module decides, once per program,
which launches go to the second lane and where the waits are.

Dependencies are taken from the memory the launches touch - the device allocations behind their buffers,
which several buffers share when their lifetimes do not overlap - not from the jaxpr: launch j depends on an
earlier launch i when one of them may write an allocation the other touches (read after write, write after
read, write after write). Every launch says which of its arrays it writes (kernels.Launch.written).

The plan is a list schedule over two lanes with an estimate of each launch's duration (its algorithmic
FLOP and bytes against typical rates, plus a fixed cost): a launch goes to the second lane when it
could start clearly sooner there than behind its predecessors on the first lane. The results of a program
do not depend on the plan; its launches are the same ones.

Measured on MI355X (device time of a replayed step, HIP events): 64 small launches in one stream 141 us; the
same with one of them on the second lane (one fork, one join) 165 us; alternating lanes with a wait before
every launch 869 us, i.e. about 12 us per dependency between the streams, with events that release to device
scope only (hipEventReleaseToDevice; 56 us for fork and join with default events). With the plans below,
gather + scatter-add went from 164 to 190 us (measured while the scatter-add had three index launches in front of
its data pass: three stream dependencies; the gather and the data pass are both bound by HBM and gain nothing from
running side by side, only the 23 us of index passes could hide), ResNet-50 at batch 64 from 4.96 to 5.06 ms (the first block of every stage: conv1 beside the
projection; storage reuse makes conv2 wait for the projection's reads), the MLP training step from 147 to
212 us. JaxprInterpreter(two_lanes=True) therefore has to be asked for; the default is one in-order stream.
'''
import typing as tp

from . import fusion

#a launch moves only if it could start at least this much sooner on the other lane (a cross-lane wait costs a few
#microseconds on the host and on the device)
MIN_GAIN_SECONDS = 8e-6
#estimate of a launch's duration: the larger of its arithmetic and its memory time at typical rates, plus a fixed cost
TYPICAL_FLOPS, TYPICAL_BYTES_PER_SECOND, FIXED_SECONDS, WAIT_SECONDS = 100e12, 5e12, 4e-6, 4e-6


class LanePlan(tp.NamedTuple):
    lane: tp.List[int]            #per launch: 0 or 1
    wait: tp.List[bool]           #per launch: its lane waits for the other lane before it is issued
    depends_on: tp.List[tp.List[int]]


def estimated_seconds(launch) -> float:
    members = launch.members or (launch,)
    flops = sum(m.flops for m in members)
    nbytes = sum(m.bytes_moved for m in members)
    return max(flops / TYPICAL_FLOPS, nbytes / TYPICAL_BYTES_PER_SECOND) + FIXED_SECONDS


def touched_and_written(op, launch) -> tp.Tuple[tp.Set[int], tp.Set[int]]:
    '''The device allocations a launch touches and the ones it may write, as ids of the pool's tensors.'''
    def tensors(buffers):
        return {id(b.tensor) for b in buffers if b is not None and b.tensor is not None}
    if launch.members:
        #a batch of small launches: every member's kernel writes its first array and reads the others
        touched = tensors(b for m in launch.members for b, _ in m.buffers)
        written = tensors(m.buffers[0][0] for m in launch.members if m.buffers)
        return touched, written
    #chains and convolutions know their results (a convolution may store a second one from its epilogue); every other
    #kernel says which of its arrays it writes
    if op.chain is not None or op.conv is not None:
        written = tensors(fusion._writes(op))
    else:
        written = tensors(launch.buffers[i][0] for i in launch.written if i < len(launch.buffers))
    return tensors(b for b, _ in launch.buffers) | written, written


def dependencies(ops, launches) -> tp.List[tp.List[int]]:
    '''For every launch the earlier launches it must not overtake.'''
    sets = [touched_and_written(op, launch) for op, launch in zip(ops, launches)]
    result = []
    for j, (touched_j, written_j) in enumerate(sets):
        deps = [i for i in range(j) if (sets[i][1] & touched_j) or (written_j & sets[i][0])]
        result.append(deps)
    return result


def plan(ops, launches) -> LanePlan:
    n = len(launches)
    deps = dependencies(ops, launches)
    lane, wait = [0] * n, [False] * n
    if n < 3:
        return LanePlan(lane, wait, deps)
    finish   = [0.0] * n
    lane_end = [0.0, 0.0]                     #when each lane's last launch ends (estimated)
    last_on  = [-1, -1]                       #the last launch issued on each lane
    seen     = [-1, -1]                       #per lane: the latest launch of the OTHER lane it has waited for
    for k, launch in enumerate(launches):
        seconds = estimated_seconds(launch)
        ready   = max((finish[i] for i in deps[k]), default=0.0)
        def start_on(l):
            needs_wait = any(lane[i] != l and i > seen[l] for i in deps[k])
            return max(lane_end[l], ready) + (WAIT_SECONDS if needs_wait else 0.0), needs_wait
        start0, wait0 = start_on(0)
        start1, wait1 = start_on(1)
        #the second lane is for launches that something on the first lane would hold up for no reason
        choose1 = start1 + MIN_GAIN_SECONDS <= start0
        l = 1 if choose1 else 0
        lane[k], wait[k] = l, (wait1 if l else wait0)
        start = start1 if l else start0
        if wait[k]:
            seen[l] = last_on[1 - l]           #the wait covers everything issued on the other lane so far
        finish[k]   = start + seconds
        lane_end[l] = finish[k]
        last_on[l]  = k
    if not any(lane):
        wait = [False] * n
    return LanePlan(lane, wait, deps)


def check(plan_: LanePlan) -> None:
    '''Every dependency is ordered by the plan: same lane (in-order), or a wait on the dependent's lane, at or after
    the dependency and at or before the dependent, that covers it. Raises AssertionError otherwise.'''
    n = len(plan_.lane)
    for k in range(n):
        for i in plan_.depends_on[k]:
            if plan_.lane[i] == plan_.lane[k]:
                continue
            #a wait of lane[k] issued for some launch w with i < w <= k covers i (recorded order is issue order)
            covered = any(plan_.wait[w] and plan_.lane[w] == plan_.lane[k] for w in range(i + 1, k + 1))
            assert covered, f'launch {k} (lane {plan_.lane[k]}) may overtake launch {i} (lane {plan_.lane[i]})'
