"""The sampler's bookkeeping on the host: the distinct ids of a request's penalty window, kept up
to date token by token, against gathering them anew from the context every step."""
import random


def test_the_penalty_window_kept_up_to_date_equals_the_window_gathered_anew():
    from spite_amd.sampling.sampler import _Window
    rnd = random.Random(1)
    for n in (0, 1, 5, 64):
        w = _Window(n)
        ctx = [rnd.randrange(20) for _ in range(rnd.randrange(0, 100))]
        for step in range(300):
            win = ctx if n == 0 or n >= len(ctx) else ctx[-n:]
            assert w.ids(ctx, 18) == sorted({t for t in win if 0 <= t < 18}), (n, step)
            ctx.extend(rnd.randrange(20) for _ in range(rnd.choice([1, 1, 1, 2, 70])))     # a token, or a long jump
        # another, shorter context under the same key starts afresh
        assert w.ids([3, 3, 25, 1], 18) == ([1, 3] if n != 1 else [1])
