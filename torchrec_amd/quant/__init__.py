from torchrec_amd.quant.embedding_modules import (  # noqa: F401
    EmbeddingBagCollection,
    EmbeddingCollection,
    FeatureProcessedEmbeddingBagCollection,
    QuantManagedCollisionEmbeddingCollection,
    quant_prep_customize_row_alignment,
    quant_prep_enable_cache_features_order,
    quant_prep_enable_quant_state_dict_split_scale_bias,
    quant_prep_enable_quant_state_dict_split_scale_bias_for_types,
    quant_prep_enable_register_tbes,
    quantize_state_dict,
)
