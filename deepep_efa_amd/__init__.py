"""MI355X-native MoE token dispatch/combine hot path behind the deep_ep.Buffer API."""
