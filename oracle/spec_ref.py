"""CPU restatement of the reference's prompt-lookup speculative decoding tasks.  TEST INFRASTRUCTURE: only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline may import this; the product never does.

Restated from
  * find_ngram_partial_kernel   include/mirage/persistent_kernel/tasks/speculative_decoding/prompt_lookup.cuh:22-100
  * find_ngram_global_kernel    .../prompt_lookup.cuh:102-140
  * target_verify_greedy_kernel .../target_verify.cuh:21-62
  * how the runtime calls them  src/kernel/task_register.cc:1713-1716 (input_token_num = step + 1), :1745-1752 (step),
                                :1778-1782 (new tokens land at tokens + step + 1, the count in new_token_nums)
  * how the step advances       include/mirage/persistent_kernel/persistent_kernel.cuh:541-552 (step += new_token_nums)

Pinned by tests/test_spec_decode.py against (a) the two scenarios of the reference's own test
(tests/runtime_python/test_prompt_lookup.py: a planted n-gram whose five followers must come back behind the regular
token; no earlier occurrence -> -1 everywhere), (b) a brute-force "earliest earlier occurrence" search on random
sequences over a tiny vocabulary, (c) the invariant that greedy speculative decoding reproduces plain greedy decoding
token for token for any deterministic next-token function.

One deliberate difference: a match is decided on the real tokens idx .. idx + N - 1.  The reference compares against a
shared-memory window whose last N - 1 entries are loaded only when they lie below T - N (prompt_lookup.cuh:62-72), so for
candidate positions idx > T - 2 N it reads entries it never set; what it returns there is undefined.
"""
LLONG_MAX = (1 << 63) - 1
NUM_THREADS = 128  # threads per task of the reference's worker block


def find_ngram_partial(tokens, input_token_num: int, ngram_size: int, num_tasks: int):
    """out[task] = the smallest idx in the task's share of [0, input_token_num - ngram_size) at which the last
    `ngram_size` of the first `input_token_num` tokens occur, LLONG_MAX if none.  Position idx belongs to task
    (idx // 128) % num_tasks (thread t of task k looks at t + 128 k + 128 num_tasks * round)."""
    out = [LLONG_MAX] * num_tasks
    if input_token_num <= ngram_size:
        return out  # (the reference returns before writing anything)
    ngram = [int(x) for x in tokens[input_token_num - ngram_size:input_token_num]]
    total = input_token_num - ngram_size
    per_round = num_tasks * NUM_THREADS
    for task in range(num_tasks):
        best, rnd = LLONG_MAX, 0
        while rnd * per_round < total and best == LLONG_MAX:  # the block stops after the first round with a match
            for t in range(NUM_THREADS):
                idx = t + task * NUM_THREADS + rnd * per_round
                if idx < total and all(int(tokens[idx + i]) == ngram[i] for i in range(ngram_size)):
                    best = min(best, idx)
            rnd += 1
        out[task] = best
    return out


def find_ngram_global(partial, tokens, step: int, ngram_size: int, spec_length: int):
    """out[0] = tokens[step]; out[1 + t] = tokens[first + ngram_size + t] while that index is <= step, else -1, where
    first = min(partial) (no match: all -1)."""
    first = min(int(p) for p in partial)
    out = [int(tokens[step])]
    for t in range(spec_length):
        ci = first + ngram_size + t
        out.append(int(tokens[ci]) if first != LLONG_MAX and ci <= step else -1)
    return out


def target_verify_greedy(spec_tokens, target_tokens, num_spec_tokens: int):
    """(new_accepted_len, new_tokens): spec_tokens[0] is the newest real token, [1..] the guesses; target_tokens[i] is what
    the model sampled on row i.  Guesses are accepted while they equal the model's token of the row before; the
    accepted targets plus the first disagreeing one are the new tokens."""
    accepted = num_spec_tokens
    for i in range(num_spec_tokens):
        if int(spec_tokens[i + 1]) != int(target_tokens[i]):
            accepted = i
            break
    return accepted + 1, [int(x) for x in target_tokens[:accepted + 1]]


def prompt_lookup_rows(tokens, step: int, ngram_size: int, spec_length: int, num_tasks: int = 96):
    """The ids of a decoding request's rows in one iteration: both n-gram tasks as the runtime chains them."""
    part = find_ngram_partial(tokens, step + 1, ngram_size, num_tasks)
    return find_ngram_global(part, tokens, step, ngram_size, spec_length), part


def accepted_with_eos(spec_rows, target_rows, eos_token_id):
    """Tokens a decoding request keeps from an iteration of n = len(spec_rows) rows when an end-of-sequence token must stay
    the request's last one: target_verify_greedy's count, cut behind the first accepted EOS.  (The reference checks only the
    FIRST new token against EOS, persistent_kernel.cuh:564-566, and would run on past an EOS accepted further back.)"""
    n = len(spec_rows)
    count, new = target_verify_greedy(spec_rows, target_rows, n - 1)
    for j in range(count):
        if new[j] == eos_token_id:
            return j + 1
    return count


def speculative_greedy_decode(next_token, prompt, max_len: int, ngram_size: int, spec_length: int, eos_token_id=None):
    """Whole-sequence model of the loop: `next_token(prefix)` is a deterministic greedy model.  Returns (tokens, iterations)."""
    toks = [int(x) for x in prompt]
    iters = 0
    while len(toks) < max_len:
        step = len(toks) - 1
        n_guess = min(spec_length, max_len - 1 - len(toks))
        rows, _ = prompt_lookup_rows(toks + [0] * (spec_length + 2), step, ngram_size, spec_length)
        rows = rows[:1 + max(n_guess, 0)]
        target = []
        for j in range(len(rows)):
            prefix = toks + [r for r in rows[1:j + 1]]
            target.append(next_token(prefix) if all(r >= 0 for r in rows[1:j + 1]) else -2)
        keep = accepted_with_eos(rows, target, eos_token_id)
        toks.extend(target[:keep])
        iters += 1
        if eos_token_id is not None and toks[-1] == eos_token_id:
            break
    return toks, iters
