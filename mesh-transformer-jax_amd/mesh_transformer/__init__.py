"""MI355X-native GPT-J generate path behind the call surface of mesh-transformer-jax's
`mesh_transformer` package (transformer_shard.CausalTransformer, layers.*, sampling.*)."""
