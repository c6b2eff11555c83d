"""The reference's text checkpoints, read and written on the host.

Three layouts, all "one float per line" under section headers:

* network / trainer files (deep_rl/checkpoint/checkpoint.mojo:5-24, written by
  deep_rl/training/network.mojo:774-798): a `# mojo-rl checkpoint v1` header with `# type`,
  `# param_size`, `# state_size`, `# dtype` lines, then `params:`, `optimizer_state:` and an
  optional `metadata:` section of key=value lines;
* the discrete PPO agent (deep_agents/ppo/ppo.mojo:3926-3980): the same header style with
  `# actor_param_size` / `# critic_param_size`, sections `actor_params:`,
  `actor_optimizer_state:`, `critic_params:`, `critic_optimizer_state:`, `metadata:`;
* the continuous PPO agent (deep_agents/ppo/ppo_continuous.mojo:493-523): bracketed sections
  `[AGENT_TYPE]`, `[HYPERPARAMETERS]`, `[ACTOR_PARAMS]`, `[ACTOR_STATE]`, `[CRITIC_PARAMS]`,
  `[CRITIC_STATE]`.

Readers follow the reference's readers line for line in what they accept and what they do with
short or damaged files (noted at each function).  Numbers are written as the shortest decimal
that reads back to the same double (every float32 is exactly a double, so a file written here
restores the float32 bit patterns through `atof`, the reference's parser, and through `float()`
here).  Adam's step count is not part of any of the formats, as in the reference.
"""
import numpy as np

HEADER_LINE = "# mojo-rl checkpoint v1"


class CheckpointHeader:
    """checkpoint.mojo:32-71."""

    def __init__(self, version=1, checkpoint_type="network", param_size=0, state_size=0, dtype_str="float32"):
        self.version, self.checkpoint_type = version, checkpoint_type
        self.param_size, self.state_size, self.dtype_str = param_size, state_size, dtype_str


def _fmt(x):
    return repr(float(x))


def _floats(values):
    """Host float64 list of a tensor / array / sequence (float32 values widen exactly)."""
    if hasattr(values, "detach"):
        values = values.detach().cpu().numpy()
    return np.asarray(values, dtype=np.float64).reshape(-1).tolist()


def write_checkpoint_header(checkpoint_type, param_size, state_size):
    """checkpoint.mojo:74-93."""
    return "%s\n# type: %s\n# param_size: %d\n# state_size: %d\n# dtype: float32\n" % (
        HEADER_LINE, checkpoint_type, param_size, state_size)


def write_float_section(section_name, data):
    """checkpoint.mojo:96-130: the header line, then one value per line."""
    vals = _floats(data)
    return section_name + "\n" + "".join(_fmt(v) + "\n" for v in vals)


def write_metadata_section(metadata):
    """checkpoint.mojo:133-145: `metadata` is a list of "key=value" strings."""
    return "metadata:\n" + "".join(m + "\n" for m in metadata)


def save_checkpoint_file(filepath, content):
    with open(filepath, "w") as f:
        f.write(content)


def read_checkpoint_file(filepath):
    with open(filepath, "r") as f:
        return f.read()


def split_lines(content):
    """checkpoint.mojo:160-182: split at "\\n"; a last line without a newline still counts, an
    empty tail does not."""
    lines = content.split("\n")
    if lines and lines[-1] == "":
        lines.pop()
    return lines


def parse_checkpoint_header(content):
    """checkpoint.mojo:185-222: header fields up to the `params:` line."""
    h = CheckpointHeader()
    for line in split_lines(content):
        if line.startswith("# mojo-rl checkpoint v"):
            h.version = int(line[len("# mojo-rl checkpoint v"):])
        elif line.startswith("# type: "):
            h.checkpoint_type = line[len("# type: "):]
        elif line.startswith("# param_size: "):
            h.param_size = int(line[len("# param_size: "):])
        elif line.startswith("# state_size: "):
            h.state_size = int(line[len("# state_size: "):])
        elif line.startswith("# dtype: "):
            h.dtype_str = line[len("# dtype: "):]
        elif line == "params:":
            break
    return h


def find_section_start(lines, section_name):
    """checkpoint.mojo:225-239: index of the line after the header, -1 if there is none."""
    for i, line in enumerate(lines):
        if line == section_name:
            return i + 1
    return -1


def read_float_section(content, section_name, size):
    """checkpoint.mojo:242-318: `size` float32 values; a missing section, a line past the end of
    the file, an empty line, a comment or another section header all read as 0."""
    lines = split_lines(content) if isinstance(content, str) else content
    out = np.zeros(size, dtype=np.float32)
    start = find_section_start(lines, section_name)
    if start < 0:
        return out
    for i in range(size):
        k = start + i
        if k >= len(lines):
            break
        line = lines[k]
        if len(line) == 0 or line.startswith("#") or line.endswith(":"):
            continue
        out[i] = np.float32(float(line))
    return out


def read_metadata_section(content):
    """checkpoint.mojo:321-345: the key=value lines after `metadata:` up to the next comment or
    section header (empty lines skipped)."""
    lines = split_lines(content)
    start = find_section_start(lines, "metadata:")
    out = []
    if start < 0:
        return out
    for line in lines[start:]:
        if len(line) == 0:
            continue
        if line.startswith("#") or line.endswith(":"):
            break
        if "=" in line:
            out.append(line)
    return out


def get_metadata_value(metadata, key):
    """checkpoint.mojo:348-365: "" when the key is absent."""
    prefix = key + "="
    for m in metadata:
        if m.startswith(prefix):
            return m[len(prefix):]
    return ""


# ---------------------------------------------------------------- Network (network.mojo:774-835)

def save_network(network, filepath):
    p = network.model.PARAM_SIZE
    s = p * network.optimizer.STATE_PER_PARAM
    content = write_checkpoint_header("network", p, s)
    content += write_float_section("params:", network.params)
    content += write_float_section("optimizer_state:", network.optimizer_state)
    save_checkpoint_file(filepath, content)


def load_network(network, filepath):
    """A size mismatch is a warning, as in the reference: what the file has is loaded, the rest
    reads as zeros."""
    p = network.model.PARAM_SIZE
    s = p * network.optimizer.STATE_PER_PARAM
    content = read_checkpoint_file(filepath)
    header = parse_checkpoint_header(content)
    if header.param_size != p:
        print("Warning: checkpoint param_size (%d) != network PARAM_SIZE (%d)" % (header.param_size, p))
    lines = split_lines(content)
    _to_device(network.params, read_float_section(lines, "params:", p))
    _to_device(network.optimizer_state, read_float_section(lines, "optimizer_state:", s))


def _to_device(dst, host):
    import torch
    dst.copy_(torch.from_numpy(np.ascontiguousarray(host, dtype=np.float32)))


# ---------------------------------------------------------------- discrete PPO agent

_DISCRETE_FLOAT_KEYS = ("gamma", "gae_lambda", "clip_epsilon", "actor_lr", "critic_lr", "entropy_coef",
                        "value_loss_coef")


def save_ppo_agent(agent, filepath):
    """ppo.mojo:3926-3980."""
    ap, cp = agent.actor.model.PARAM_SIZE, agent.critic.model.PARAM_SIZE
    content = "%s\n# type: ppo_agent\n# actor_param_size: %d\n# critic_param_size: %d\n" % (HEADER_LINE, ap, cp)
    content += write_float_section("actor_params:", agent.actor.params)
    content += write_float_section("actor_optimizer_state:", agent.actor.optimizer_state)
    content += write_float_section("critic_params:", agent.critic.params)
    content += write_float_section("critic_optimizer_state:", agent.critic.optimizer_state)
    meta = ["%s=%s" % (k, _fmt(getattr(agent, k))) for k in _DISCRETE_FLOAT_KEYS]
    meta += ["num_epochs=%d" % agent.num_epochs, "minibatch_size=%d" % agent.minibatch_size,
             "normalize_advantages=%s" % ("True" if agent.normalize_advantages else "False"),
             "target_kl=" + _fmt(agent.target_kl), "max_grad_norm=" + _fmt(agent.max_grad_norm),
             "train_step_count=%d" % agent.train_step_count]
    content += write_metadata_section(meta)
    save_checkpoint_file(filepath, content)


def _strict_section(lines, name, size):
    """ppo.mojo:3997-4022: every one of the `size` lines after the header must parse (a short or
    damaged file raises, as `atof` does there)."""
    start = find_section_start(lines, name)
    if start < 0 or start + size > len(lines):
        raise ValueError("checkpoint section %r is missing or shorter than %d values" % (name, size))
    return np.array([float(x) for x in lines[start:start + size]], dtype=np.float64).astype(np.float32)


def load_ppo_agent(agent, filepath):
    """ppo.mojo:3982-4055: the four arrays, then every known key of the metadata section."""
    ap, cp = agent.actor.model.PARAM_SIZE, agent.critic.model.PARAM_SIZE
    spp = agent.actor.optimizer.STATE_PER_PARAM
    lines = split_lines(read_checkpoint_file(filepath))
    _to_device(agent.actor.params, _strict_section(lines, "actor_params:", ap))
    _to_device(agent.actor.optimizer_state, _strict_section(lines, "actor_optimizer_state:", ap * spp))
    _to_device(agent.critic.params, _strict_section(lines, "critic_params:", cp))
    _to_device(agent.critic.optimizer_state, _strict_section(lines, "critic_optimizer_state:", cp * spp))
    start = find_section_start(lines, "metadata:")
    for line in lines[start:] if start >= 0 else []:
        key, sep, val = line.partition("=")
        if not sep:
            continue
        if key in _DISCRETE_FLOAT_KEYS or key in ("target_kl", "max_grad_norm"):
            setattr(agent, key, float(val))
        elif key in ("num_epochs", "minibatch_size", "train_step_count"):
            setattr(agent, key, int(val))
        elif key == "normalize_advantages":
            agent.normalize_advantages = val == "True"
    agent.actor.optimizer.lr, agent.critic.optimizer.lr = agent.actor_lr, agent.critic_lr


# ---------------------------------------------------------------- continuous PPO agent

def save_ppo_continuous_agent(agent, filepath):
    """ppo_continuous.mojo:493-523."""
    content = "[AGENT_TYPE]\nDeepPPOContinuousAgent\n[HYPERPARAMETERS]\n"
    for k in ("gamma", "gae_lambda", "clip_epsilon", "actor_lr", "critic_lr", "entropy_coef"):
        content += "%s=%s\n" % (k, _fmt(getattr(agent, k)))
    content += "train_step_count=%d\n" % agent.train_step_count
    content += write_float_section("[ACTOR_PARAMS]", agent.actor.params)
    content += write_float_section("[ACTOR_STATE]", agent.actor.optimizer_state)
    content += write_float_section("[CRITIC_PARAMS]", agent.critic.params)
    content += write_float_section("[CRITIC_STATE]", agent.critic.optimizer_state)
    save_checkpoint_file(filepath, content)


def _lenient_section(lines, name, current):
    """ppo_continuous.mojo:536-590: values are taken line by line until the next bracketed header
    or the end of the file; a line that does not parse leaves its slot as it was; a missing
    section leaves everything as it was.  Returns the new host array."""
    out = np.array(_floats(current), dtype=np.float64).astype(np.float32)
    idx = find_section_start(lines, name)
    if idx < 0:
        return out
    for i in range(out.shape[0]):
        if idx >= len(lines) or lines[idx].startswith("["):
            break
        try:
            out[i] = np.float32(float(lines[idx]))
        except ValueError:
            pass
        idx += 1
    return out


def load_ppo_continuous_agent(agent, filepath):
    """ppo_continuous.mojo:525-604.  A missing or empty file is reported and ignored; of the
    hyperparameters only train_step_count is restored (the scan starts one line into the section,
    which skips `gamma=`)."""
    try:
        content = read_checkpoint_file(filepath)
    except FileNotFoundError:
        content = ""
    if len(content) == 0:
        print("No checkpoint found at:", filepath)
        return
    lines = split_lines(content)
    for net, pname, sname in ((agent.actor, "[ACTOR_PARAMS]", "[ACTOR_STATE]"),
                              (agent.critic, "[CRITIC_PARAMS]", "[CRITIC_STATE]")):
        _to_device(net.params, _lenient_section(lines, pname, net.params))
        _to_device(net.optimizer_state, _lenient_section(lines, sname, net.optimizer_state))
    start = find_section_start(lines, "[HYPERPARAMETERS]")
    if start >= 0:
        idx = start + 1
        while idx < len(lines) and not lines[idx].startswith("["):
            if lines[idx].startswith("train_step_count="):
                try:
                    agent.train_step_count = int(float(lines[idx][len("train_step_count="):]))
                except ValueError:
                    pass
            idx += 1
    print("Checkpoint loaded from:", filepath)
