"""Step plans (bkv_step_plan_*): a decode step whose positions and cut into work-groups live in
device memory, so that the launches of one token can be captured into a graph once and replayed.
The analogue of the reference's contract test crates/breccia-kernels/tests/batching.rs:27-88
(batched == unbatched, bit for bit): the replayed steps against bkv_decode_step called token by
token on a twin pool -- identical pool bytes, identical output bits -- and against the oracle."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer, Graph, StepPlan, Stream, device_sync
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from test_gpu_attn import fill

pytestmark = pytest.mark.gpu


def grow(tw, lens, rng, order):
    tw.pool.set_free_order(order)
    seqs = [tw.pool.seq_create() for _ in lens]
    for s, n in zip(seqs, lens):
        fill(tw, s, n, rng, chunk=1024)
    return seqs


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_captured_token_replayed_32_times_equals_eager_steps(layout):
    n_layers, n_tok, n_q, n_kv = 12, 32, 16, 2
    lens = [700, 15, 2049, 330]            # a page edge inside the horizon for every sequence
    rng = np.random.Generator(np.random.PCG64(9300 + layout))
    order = rng.permutation(400).astype(np.int32)
    st = Stream()
    with Twin(n_layers=n_layers, n_pages=400, layout=layout, max_seqs=8, max_pages_per_seq=160) as eager, \
            Twin(n_layers=n_layers, n_pages=400, layout=layout, max_seqs=8, max_pages_per_seq=160) as replay:
        # the same history in layer 0 of both pools (the other layers start empty but for the new rows)
        rng_a = np.random.Generator(np.random.PCG64(77))
        rng_b = np.random.Generator(np.random.PCG64(77))
        seqs_e = grow(eager, lens, rng_a, order)
        seqs_r = grow(replay, lens, rng_b, order)
        assert seqs_e == seqs_r
        n = len(lens)
        for s, c in zip(seqs_e, lens):
            eager.pool.seq_reserve(s, c + n_tok + 1)
        for s, c in zip(seqs_r, lens):
            replay.pool.seq_reserve(s, c + n_tok + 1)
        # inputs of every (token, layer): new rows and queries
        kn = rng.standard_normal((n_tok, n_layers, n, n_kv, 256)).astype(np.float32)
        vn = rng.standard_normal((n_tok, n_layers, n, n_kv, 256)).astype(np.float32)
        q = rng.standard_normal((n_tok, n_layers, n, n_q, 256)).astype(np.float32)
        gate = rng.standard_normal((n, n_q, 256)).astype(np.float32)
        per_layer = n * n_kv * 256 * 4
        kd, vd = DeviceBuffer(n_layers * per_layer), DeviceBuffer(n_layers * per_layer)
        qd, od = DeviceBuffer(n_layers * n * n_q * 256 * 4), DeviceBuffer(n_layers * n * n_q * 256 * 4)
        gd = DeviceBuffer.from_numpy(gate)
        q_layer = n * n_q * 256 * 4

        # ---- eager: bkv_decode_step per (token, layer) --------------------------------------
        want = np.zeros((n_tok, n_layers, n, n_q, 256), dtype=np.float32)
        for t in range(n_tok):
            kd.upload(kn[t]), vd.upload(vn[t]), qd.upload(q[t])
            pos = [c + t for c in lens]
            for layer in range(n_layers):
                eager.pool.decode_step(layer, seqs_e, pos, kd.at(layer * per_layer), vd.at(layer * per_layer), n_q,
                                       qd.at(layer * q_layer), od.at(layer * q_layer), 1.0 / 16.0, gate_dev=gd,
                                       gate_seq_stride=n_q * 256, gate_head_stride=256)
            device_sync()
            want[t] = od.download(np.float32).reshape(n_layers, n, n_q, 256)

        # ---- one token captured, replayed n_tok times ---------------------------------------
        # checked for one cell more than the tokens to come: the advance that ends the last token stays inside
        plan = StepPlan(replay.pool, seqs_r, lens, n_tok + 1, n_q, stream=st)
        g = Graph(st)
        for layer in range(n_layers):
            plan.decode(layer, kd.at(layer * per_layer), vd.at(layer * per_layer), qd.at(layer * q_layer),
                        od.at(layer * q_layer), 1.0 / 16.0, gate_dev=gd, gate_seq_stride=n_q * 256,
                        gate_head_stride=256, stream=st)
        plan.advance(st)
        g.end()
        got = np.zeros_like(want)
        for t in range(n_tok):
            # eager work and synchronisation between the replays: this token's inputs
            kd.upload(kn[t], st), vd.upload(vn[t], st), qd.upload(q[t], st)
            g.launch(st)
            st.sync()
            got[t] = od.download(np.float32, stream=st).reshape(n_layers, n, n_q, 256)
        pos, steps, status = plan.state(st)
        assert steps == n_tok and status == 0 and list(pos) == [c + n_tok for c in lens]
        for t in range(n_tok):
            assert np.array_equal(want[t].view(np.uint32), got[t].view(np.uint32)), "token %d differs" % t
        for layer in (0, 5, n_layers - 1):
            assert np.array_equal(eager.pool.read_layer(layer, 0), replay.pool.read_layer(layer, 0))
            assert np.array_equal(eager.pool.read_layer(layer, 1), replay.pool.read_layer(layer, 1))

        # one more advance would pass the cells the plan was checked for: nothing moves, the status says so
        before_k = replay.pool.read_layer(3, 0)
        plan.advance(st)
        pos2, steps2, status2 = plan.state(st)
        assert status2 == 1 and steps2 == n_tok and list(pos2) == list(pos)
        assert np.array_equal(before_k, replay.pool.read_layer(3, 0))

        # the oracle, on layer 0 (the layer with the history), last token
        t = n_tok - 1
        for i, s in enumerate(seqs_r):
            img = replay.images[0]
            table = replay.pool.block_table(s)
            for tt in range(n_tok):
                assert img.append(table, lens[i] + tt, kn[tt, 0, i][None], vn[tt, 0, i][None]) == 0
            _, rel = check_attn(got[t, 0, i], replay.oracle_attend(0, s, lens[i] + t, q[t, 0, i], n_q, gate=gate[i]),
                                "replayed token %d, sequence %d" % (t, i))
            assert rel <= REF_BAR_MAX_REL, (i, rel)
        g.destroy()
        plan.destroy()
        for b in (kd, vd, qd, od, gd):
            b.free()
    st.close()


def test_a_plan_made_on_one_stream_and_driven_from_others_needs_no_host_synchronisation():
    # The plan's descriptor is uploaded on the stream of its creation, behind whatever that stream
    # still has to do (here: bulk appends and the scatter of freshly reserved pages' table entries);
    # decode arrives on a second stream and advance on a third, with no host synchronisation in
    # between.  The library orders them (events, on the device): outputs and pool bytes equal the eager
    # steps' of a twin pool, bit for bit.
    n_q, lens, n_tok = 16, [333, 47], 5
    rng = np.random.Generator(np.random.PCG64(9400))
    a, b, c = Stream(), Stream(), Stream()
    with Twin(n_pages=2200, max_seqs=8, max_pages_per_seq=1100) as eager, \
            Twin(n_pages=2200, max_seqs=8, max_pages_per_seq=1100) as planned:
        rng_a, rng_b = np.random.Generator(np.random.PCG64(5)), np.random.Generator(np.random.PCG64(5))
        order = rng.permutation(2200).astype(np.int32)
        seqs = grow(eager, lens, rng_a, order)
        assert grow(planned, lens, rng_b, order) == seqs
        kn = rng.standard_normal((n_tok, 2, 2, 256)).astype(np.float32)
        vn = rng.standard_normal((n_tok, 2, 2, 256)).astype(np.float32)
        q = rng.standard_normal((n_tok, 2, n_q, 256)).astype(np.float32)
        kd, vd, qd = DeviceBuffer.from_numpy(kn), DeviceBuffer.from_numpy(vn), DeviceBuffer.from_numpy(q)
        od = DeviceBuffer(q.nbytes)
        step_kv, step_q = 2 * 2 * 256 * 4, 2 * n_q * 256 * 4
        want = np.zeros_like(q)
        for t in range(n_tok):
            for s, n in zip(seqs, lens):
                eager.pool.seq_reserve(s, n + t + 1)
            eager.pool.decode_step(0, seqs, [n + t for n in lens], kd.at(t * step_kv), vd.at(t * step_kv), n_q,
                                   qd.at(t * step_q), od.at(t * step_q), 1.0 / 16.0)
        device_sync()
        want = od.download(np.float32).reshape(q.shape)
        od.upload(np.zeros_like(q))
        # the planned pool: a long tail of work on stream a (a third sequence filled with 16384 tokens, in
        # four calls), the step's pages reserved (their table entries pending), then the plan on stream a
        big = planned.pool.seq_create()
        planned.pool.seq_reserve(big, 16384)
        rows = DeviceBuffer.from_numpy(rng.standard_normal((4096, 2, 256)).astype(np.float32))
        for s, n in zip(seqs, lens):
            planned.pool.seq_reserve(s, n + n_tok + 1)
        for i in range(4):
            planned.pool.append(0, [big], [4096 * i], [4096], rows, rows, a)
        plan = StepPlan(planned.pool, seqs, lens, n_tok + 1, n_q, stream=a)
        for t in range(n_tok):
            plan.decode(0, kd.at(t * step_kv), vd.at(t * step_kv), qd.at(t * step_q), od.at(t * step_q), 1.0 / 16.0,
                        stream=b)
            plan.advance(c)
        pos, steps, status = plan.state(b)
        assert steps == n_tok and status == 0 and pos.tolist() == [n + n_tok for n in lens]
        got = od.download(np.float32).reshape(q.shape)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        device_sync()
        planned.pool.seq_free(big)
        for s in seqs:
            ge, gp = eager.pool.gather(0, s, 0, lens[seqs.index(s)] + n_tok), planned.pool.gather(0, s, 0, lens[seqs.index(s)] + n_tok)
            assert np.array_equal(ge[0].view(np.uint32), gp[0].view(np.uint32))
            assert np.array_equal(ge[1].view(np.uint32), gp[1].view(np.uint32))
        plan.destroy()
        for x in (kd, vd, qd, od, rows):
            x.free()


def test_plan_creation_checks_the_whole_horizon():
    with Twin(n_pages=32, max_seqs=4) as tw:
        a, b = tw.pool.seq_create(), tw.pool.seq_create()
        tw.pool.seq_reserve(a, 40)
        tw.pool.seq_reserve(b, 40)
        with pytest.raises(BkvError) as ei:          # cells 30..49 of a: only 40 reserved
            StepPlan(tw.pool, [a], [30], 20, 16)
        assert ei.value.status == L.ERR_RANGE
        with pytest.raises(BkvError) as ei:          # the same sequence twice
            StepPlan(tw.pool, [a, a], [10, 11], 4, 16)
        assert ei.value.status == L.ERR_INVALID
        child = tw.pool.seq_fork(a, 35)              # a's third page is now shared
        with pytest.raises(BkvError) as ei:
            StepPlan(tw.pool, [a], [30], 8, 16)
        assert ei.value.status == L.ERR_STATE
        tw.pool.seq_free(child)
        plan = StepPlan(tw.pool, [a, b], [30, 20], 10, 16)
        with pytest.raises(BkvError) as ei:          # a plan points into its pool
            tw.pool.destroy()
        assert ei.value.status == L.ERR_STATE
        plan.destroy()


def test_a_plan_whose_sequences_changed_is_refused_at_the_next_call():
    """Between creation and the last use the plan's sequences are to be left alone; a host call that
    enqueues the plan's kernels looks again, and a sequence that was forked (its page now shared),
    truncated or freed since is an error before anything is launched."""
    rng = np.random.Generator(np.random.PCG64(9400))
    with Twin(n_pages=32, max_seqs=4) as tw:
        a, b = tw.pool.seq_create(), tw.pool.seq_create()
        fill(tw, a, 30, rng)
        fill(tw, b, 20, rng)
        tw.pool.seq_reserve(a, 40)
        tw.pool.seq_reserve(b, 40)
        plan = StepPlan(tw.pool, [a, b], [30, 20], 10, 16)
        kn = DeviceBuffer.from_numpy(rng.standard_normal((2, 2, 256)).astype(np.float32))
        q = DeviceBuffer.from_numpy(rng.standard_normal((2, 16, 256)).astype(np.float32))
        out = DeviceBuffer(2 * 16 * 256 * 4)
        plan.decode(0, kn, kn, q, out, 1.0 / 16.0)      # as made: fine
        device_sync()
        before = tw.pool.read_layer(0, 0).copy()
        child = tw.pool.seq_fork(a, 35)                  # a's third page is shared now
        with pytest.raises(BkvError) as ei:
            plan.decode(0, kn, kn, q, out, 1.0 / 16.0)
        assert ei.value.status == L.ERR_STATE
        tw.pool.seq_free(child)
        plan.decode(0, kn, kn, q, out, 1.0 / 16.0)      # sole holder again
        tw.pool.seq_truncate(b, 25)                      # cells 25..29 of b are no longer reserved
        with pytest.raises(BkvError) as ei:
            plan.decode(0, kn, kn, q, out, 1.0 / 16.0)
        assert ei.value.status == L.ERR_STATE
        tw.pool.seq_reserve(b, 40)
        tw.pool.seq_free(a)
        with pytest.raises(BkvError) as ei:
            plan.decode(0, kn, kn, q, out, 1.0 / 16.0)
        assert ei.value.status == L.ERR_STATE
        device_sync()
        # the refused calls wrote nothing (the two accepted ones rewrote the same row)
        assert np.array_equal(before, tw.pool.read_layer(0, 0))
        plan.destroy()
        for x in (kn, q, out):
            x.free()


def test_the_device_cuts_a_large_ragged_batch_as_the_host_does():
    """The advance kernel re-plans on the device with the host planner's arithmetic: over 40 advances
    of 64 sequences of very different lengths (page edges crossed all the time, the cut changing with
    them), a step replayed from the plan returns the bits of bkv_decode_step at the same positions."""
    n, n_q, n_tok = 64, 16, 40
    rng = np.random.Generator(np.random.PCG64(9400))
    lens = [int(x) for x in rng.integers(0, 70, size=40)] + [int(x) for x in rng.integers(200, 3000, size=24)]
    order = rng.permutation(4096).astype(np.int32)
    st = Stream()
    with Twin(n_pages=4096, max_seqs=64, max_pages_per_seq=200) as a, \
            Twin(n_pages=4096, max_seqs=64, max_pages_per_seq=200) as b:
        seqs = None
        for tw in (a, b):
            r2 = np.random.Generator(np.random.PCG64(5))
            tw.pool.set_free_order(order)
            ss = [tw.pool.seq_create() for _ in lens]
            for s, c in zip(ss, lens):
                if c:
                    fill(tw, s, c, r2, chunk=1024)
                tw.pool.seq_reserve(s, c + n_tok + 1)
            assert seqs is None or seqs == ss
            seqs = ss
        kn = rng.standard_normal((n_tok, n, 2, 256)).astype(np.float32)
        q = rng.standard_normal((n, n_q, 256)).astype(np.float32)
        kd, qd = DeviceBuffer(kn[0].nbytes), DeviceBuffer.from_numpy(q)
        oe, op = DeviceBuffer(q.nbytes), DeviceBuffer(q.nbytes)
        plan = StepPlan(b.pool, seqs, lens, n_tok + 1, n_q, stream=st)
        for t in range(n_tok):
            kd.upload(kn[t])
            device_sync()
            a.pool.decode_step(0, seqs, [c + t for c in lens], kd, kd, n_q, qd, oe, 1.0 / 16.0)
            plan.decode(0, kd, kd, qd, op, 1.0 / 16.0, stream=st)
            plan.advance(st)
            st.sync()
            device_sync()
            if t % 3 == 0 or t == n_tok - 1:
                assert np.array_equal(oe.download(np.uint32), op.download(np.uint32)), "token %d" % t
        pos, steps, status = plan.state(st)
        assert steps == n_tok and status == 0 and list(pos) == [c + n_tok for c in lens]
        assert np.array_equal(a.pool.read_layer(0, 0), b.pool.read_layer(0, 0))
        plan.destroy()
        for x in (kd, qd, oe, op):
            x.free()
    st.close()
